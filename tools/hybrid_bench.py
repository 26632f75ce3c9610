"""`bench.py --hybrid`: prefill and decode throughput of the hybrid decoder (latent attention + lightning recurrence + routed
experts) at layer sizes that resemble a real model's, beside a dense decoder (the repository's Qwen3-style stack) of equal
width, depth, head count and ACTIVE feed-forward width, and each sequence-mixing kernel alone against its roofline.

Random weights, synthetic token ids, bf16.  One JSON line on stdout; does not touch bench.py's default workload.

    python bench.py --hybrid [--hybrid-args --sizes s m --prompt 2048 --batch 32 --steps 20 --no-dense --no-kernels]
"""
from __future__ import annotations

import argparse
import json
import math
import time

import torch

HBM_TBS, MFMA_TFLOPS, VALU_TFLOPS = 8.0, 2500.0, 157.0  # spec peaks: HBM3E, dense bf16 matrix cores, fp32 vector FMA

# name -> (width, layers as a string of L = lightning / A = latent attention with own keys / B = latent attention that
#          borrows the previous A's keys, heads, head size, latent rank, rotated size, experts, top, expert ff, vocab)
SIZES = {
    "s": (1024, "LLAL", 8, 128, 256, 64, 16, 2, 1024, 32000),
    "m": (2048, "LLALLB", 16, 128, 512, 64, 32, 4, 1024, 32000),
    "l": (4096, "LLAL", 32, 128, 512, 64, 64, 8, 1024, 32000),
}


def hybrid_json(name: str) -> dict:
    W, order, H, D, R, r, E, top, ff, V = SIZES[name]
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top, "groups": {"count": 4, "keep": 2}}}
    rot = {"base": 1e6, "dims": r, "scaling": {"factor": 8.0, "fast": 32.0, "original": 4096, "slow": 1.0}}
    layers, last_a = [], None
    for i, c in enumerate(order):
        if c == "L":
            decay = [math.exp(-2.0 ** (-(1 + 7 * h / max(H - 1, 1)))) for h in range(H)]
            layers.append({"type": "lightning", "mixer": {"heads": H, "dim": D, "vdim": D, "decay": decay}, "mlp": mlp})
        else:
            m = {"heads": H, "dim": D, "rot_dim": r, "vdim": D, "kv_rank": R, "rot": rot, "scale": (D + r) ** -0.5}
            if c == "B":
                m["kv_from"] = last_a
            else:
                last_a = i
            layers.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
    return {"architecture": "Nidorax", "layers": layers, "norm": {"eps": 1e-6}, "postln_alpha": 2.0, "vocab": V, "width": W}


def dense_config(name: str):
    from mini_sglang_amd.model import ModelConfig

    W, order, H, D, R, r, E, top, ff, V = SIZES[name]
    return ModelConfig(num_layers=len(order), num_qo_heads=H, num_kv_heads=max(H // 4, 1), head_dim=D, hidden_size=W, vocab_size=V,
                       intermediate_size=top * ff, max_position=8192, tie_word_embeddings=True, name=f"dense-{name}")


def run_engine(cfg, prompt: int, batch: int, steps: int, warmup: int, device) -> dict:
    """Prefill `batch` prompts of `prompt` tokens under an 8192-token budget, then `steps` decode steps from the captured graph."""
    from mini_sglang_amd.core import SamplingParams
    from mini_sglang_amd.engine import Engine, EngineConfig
    from mini_sglang_amd.offline import OfflineRunner

    page = 16
    tokens = batch * (prompt + steps + warmup + 2 * page)
    ecfg = EngineConfig(model=cfg, dtype=torch.bfloat16, max_running_req=batch, cuda_graph_bs=[batch], page_size=page,
                        max_seq_len_override=prompt + steps + warmup + 2 * page, num_page_override=-(-tokens // page),
                        gemm_tune="heuristic", refine_in_graph=False)
    eng = Engine(ecfg, device)
    run = OfflineRunner(eng, max_extend_tokens=8192, seed=0)
    g = torch.Generator().manual_seed(0)
    sp = SamplingParams(temperature=0.0, max_tokens=steps + warmup + 1, ignore_eos=True)
    run.warmup_prefill(min(8192, batch * prompt))
    torch.cuda.synchronize(device)
    states = [run.add_request(torch.randint(0, cfg.vocab_size, (prompt,), generator=g).tolist(), sp) for _ in range(batch)]
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in run.prefill(states):
        pass
    e1.record()
    torch.cuda.synchronize(device)
    prefill_ms = e0.elapsed_time(e1)
    for _ in range(warmup):
        run.decode_step(states)
    torch.cuda.synchronize(device)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        run.decode_step(states)
    e1.record()
    torch.cuda.synchronize(device)
    decode_ms, wall_ms = e0.elapsed_time(e1) / steps, (time.perf_counter() - t0) * 1e3 / steps
    weights = eng.model.weight_bytes()
    eng.shutdown()
    del eng, run
    torch.cuda.empty_cache()
    return {"prefill_tok_s": round(batch * prompt / prefill_ms * 1e3), "decode_tok_s": round(batch / decode_ms * 1e3),
            "decode_ms_per_step": round(decode_ms, 3), "decode_wall_ms_per_step": round(wall_ms, 3), "weight_mb": weights >> 20}


def _time_us(fn, iters: int = 10) -> float:
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def kernel_rooflines(name: str, prompt: int, batch: int, device) -> dict:
    """Each sequence-mixing kernel alone at the size's shapes: microseconds, and the share of the roofline that bounds it
    (matrix cores for the products of a prompt portion, HBM for everything a decode step streams)."""
    from mini_sglang_amd import mixops

    W, order, H, D, R, r, E, top, ff, V = SIZES[name]
    bf = torch.bfloat16
    out = {}

    def rnd(*shape, dtype=bf, scale=1.0):
        return (torch.randn(shape, device=device, dtype=torch.float32) * scale).to(dtype)

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=device)

    for phase, T, reqs, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, prompt)):
        q_len = T // reqs
        cu = i32([i * q_len for i in range(reqs + 1)])
        seq = i32([ctx] * reqs)
        rows = i32(list(range(reqs)))
        slots = reqs * ctx
        table = torch.arange(slots, dtype=torch.int32, device=device).view(reqs, ctx)
        # --- latent attention over the shared latent rows
        cache, q_abs = rnd(slots, R + r), rnd(T, H, R + r, dtype=torch.float32, scale=0.1)
        o_lat = torch.empty(T, H, R, dtype=torch.float32, device=device)
        splits = mixops.latent_attn_splits(reqs, T, H, ctx) if q_len <= 16 else 1
        us = _time_us(lambda: mixops.latent_attn(o_lat, q_abs, cache, table, rows, seq, cu, reqs, R, 0.1, splits=splits))
        pairs = reqs * (q_len * (ctx - q_len) + q_len * (q_len + 1) // 2)
        flops = 2.0 * pairs * H * (2 * R + r)
        byts = reqs * ctx * (R + r) * 2 + T * H * (2 * R + r) * 4
        out[f"{phase}.latent_attn"] = {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
                                      "of_roofline": round(max(flops / us / 1e6 / MFMA_TFLOPS, byts / us / 1e6 / HBM_TBS), 4)}
        # --- lightning recurrence
        qkv = rnd(T, 4 * H * D, scale=0.5)
        state = torch.zeros(reqs, H, D, D, dtype=torch.float32, device=device)
        decay = torch.full((H,), 0.97, dtype=torch.float32, device=device)
        o = torch.empty(T, H * D, dtype=torch.float32, device=device)
        chunks = None
        if q_len >= 256:  # what the engine's metadata does for long portions: pieces of 128 tokens in parallel
            n = -(-q_len // 128)
            items = i32([[b, c * 128, min((c + 1) * 128, q_len)] for b in range(reqs) for c in range(n)]).view(-1)
            chunks = (items, i32([b * n for b in range(reqs + 1)]), reqs * n)
        us = _time_us(lambda: mixops.lightning(o, qkv, state, decay, cu, seq, rows, reqs, chunks=chunks))
        flops = 4.0 * T * H * D * D
        byts = 2 * reqs * H * D * D * 4 + T * 3 * H * D * 2 + T * H * D * 4
        out[f"{phase}.lightning"] = {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
                                    "of_roofline": round(max(flops / us / 1e6 / (MFMA_TFLOPS if phase == "prefill" else VALU_TFLOPS),
                                                             byts / us / 1e6 / HBM_TBS), 4)}
        # --- routed experts: router, bucketing, the two segmented products
        h = rnd(T, W)
        router, bias = rnd(E, W, scale=W ** -0.5), rnd(E, scale=0.01)
        up, down = rnd(E, ff, W, scale=W ** -0.5), rnd(E, W, ff, scale=ff ** -0.5)
        ids, wts = mixops.route(h, router, bias, top, 4, 2)
        seg, perm = mixops.moe_sort(ids, E)
        n = T * top
        act = torch.empty(n, ff, dtype=bf, device=device)
        y = torch.empty(T, top, W, dtype=bf, device=device)
        xr, wr, hr = rnd(T, W, dtype=torch.float32), rnd(W, scale=0.1), torch.empty(T, W, dtype=bf, device=device)
        us_r = _time_us(lambda: mixops.postnorm(xr, wr, 1e-6, y=h, alpha=2.0, x_out=xr, h_out=hr, route=(router, bias, top, 4, 2)))
        us_s = _time_us(lambda: mixops.moe_sort(ids, E))
        us_u = _time_us(lambda: mixops.gemm_nt(act, h, up, n, ff, W, lda=W, ldb=W, ldc=ff, groups=E, b_gs=ff * W, seg=seg, a_rows=perm,
                                               a_div=top, act=mixops.ACT_RELU2))
        us_d = _time_us(lambda: mixops.gemm_nt(y, act, down, n, W, ff, lda=ff, ldb=ff, ldc=W, groups=E, b_gs=W * ff, seg=seg, c_rows=perm))
        flops = 2.0 * n * ff * W
        touched = min(E, n)
        byts = touched * ff * W * 2 + n * (W + ff) * 2
        for key, us in (("experts_up", us_u), ("experts_down", us_d)):
            out[f"{phase}.{key}"] = {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
                                     "of_roofline": round(max(flops / us / 1e6 / MFMA_TFLOPS, byts / us / 1e6 / HBM_TBS), 4)}
        rb = T * W * 12 + E * W * 2  # the post-norm's traffic + the router weights once
        out[f"{phase}.postnorm_route"] = {"us": round(us_r, 1), "tb_s": round(rb / us_r / 1e6, 3), "of_roofline": round(rb / us_r / 1e6 / HBM_TBS, 4)}
        out[f"{phase}.moe_sort"] = {"us": round(us_s, 1)}
        # --- post-norm (fp32 residual in and out, 16-bit sublayer output in, 16-bit copy out)
        x = rnd(T, W, dtype=torch.float32)
        yv, wn, hh = rnd(T, W), rnd(W, scale=0.1), torch.empty(T, W, dtype=bf, device=device)
        us = _time_us(lambda: mixops.postnorm(x, wn, 1e-6, y=yv, alpha=2.0, x_out=x, h_out=hh))
        byts = T * W * (4 + 4 + 2 + 2)
        out[f"{phase}.postnorm"] = {"us": round(us, 1), "tb_s": round(byts / us / 1e6, 3), "of_roofline": round(byts / us / 1e6 / HBM_TBS, 4)}
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", nargs="*", default=["s", "m"], choices=sorted(SIZES))
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    args = ap.parse_args(argv)
    from mini_sglang_amd.hybrid import HybridConfig

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    report = {"metric": "hybrid_decoder_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
              "prompt": args.prompt, "batch": args.batch, "steps": args.steps, "sizes": {}}
    for name in args.sizes:
        entry = {"shape": dict(zip(("width", "layers", "heads", "head", "kv_rank", "rot", "experts", "top", "ff", "vocab"), SIZES[name]))}
        entry["hybrid"] = run_engine(HybridConfig.from_json(hybrid_json(name)), args.prompt, args.batch, args.steps, args.warmup, device)
        if not args.no_dense:
            entry["dense"] = run_engine(dense_config(name), args.prompt, args.batch, args.steps, args.warmup, device)
        if not args.no_kernels:
            entry["kernels"] = kernel_rooflines(name, args.prompt, args.batch, device)
        report["sizes"][name] = entry
        print(f"[hybrid bench] {name}: " + json.dumps({k: entry[k] for k in ("hybrid", "dense") if k in entry}), flush=True)
    print(json.dumps(report))


if __name__ == "__main__":
    main()
