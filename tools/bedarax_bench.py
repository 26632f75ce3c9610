"""`bench.py --bedarax`: prefill and decode throughput of the pre-norm hybrid decoder (Bedarax: windowed attention with mixed
heads + gated delta-rule layers + dense / gated-expert feed-forwards) at layer sizes that resemble a real model's, beside the
repository's closest model, the post-norm hybrid decoder (Nidorax: latent attention + lightning recurrence + routed experts) of
equal width, depth, head count, head size and expert shape, and each new kernel alone against its roofline beside its like kernel.

Random weights, synthetic token ids, bf16.  One JSON line on stdout; does not touch bench.py's default workload.

    python bench.py --bedarax [--bedarax-args --sizes s m --prompt 2048 --batch 32 --steps 20 --no-twin --no-kernels]
"""
from __future__ import annotations

import argparse
import json

import torch

from tools.hybrid_bench import HBM_TBS, MFMA_TFLOPS, VALU_TFLOPS, _time_us, run_engine

# name -> (width, layers: A = windowed attention, D = delta, C = channel_delta; heads, key heads of the attention layers, head size,
#          window, conv taps, inner size of the two-step projections, experts, top, expert ff, vocab)
SIZES = {
    "s": (1024, "DCAD", 8, 2, 128, 1024, 4, 64, 16, 2, 1024, 32000),
    "m": (2048, "DCADCA", 16, 4, 128, 2048, 4, 128, 32, 4, 1024, 32000),
}


def bedarax_json(name: str) -> dict:
    W, order, H, G, D, window, taps, rank, E, top, ff, V = SIZES[name]
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top}}
    layers = []
    for c in order:
        if c == "A":  # the attention layers carry the dense feed-forward of the ACTIVE width
            layers.append({"type": "attention", "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5,
                                                          "mask": {"size": window}, "v_mix": True}, "mlp": {"kind": "dense", "ff": top * ff}})
        else:
            layers.append({"type": "channel_delta" if c == "C" else "delta",
                           "mixer": {"heads": H, "kv_heads": H, "dim": D, "vdim": D, "conv": taps}, "mlp": moe})
    return {"architecture": "Bedarax", "layers": layers, "norm": {"eps": 1e-6}, "vocab": V, "width": W}


def bedarax_shapes(name: str) -> dict:
    W, order, H, G, D, window, taps, rank, E, top, ff, V = SIZES[name]
    return {f"l{i}.mix.{t}": (rank, W) for i, c in enumerate(order) if c == "C" for t in ("a1", "g1")}


def twin_json(name: str) -> dict:
    """The post-norm hybrid decoder of equal width, depth, heads, head size and experts: recurrent layers where this design has
    delta layers, latent attention (latent 4 x head size, 64 rotated) where it has windowed attention."""
    import math

    W, order, H, G, D, window, taps, rank, E, top, ff, V = SIZES[name]
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": E, "top": top, "groups": {"count": 4, "keep": 2}}}
    rot = {"base": 1e6, "dims": 64, "scaling": {"factor": 8.0, "fast": 32.0, "original": 4096, "slow": 1.0}}
    layers = []
    for c in order:
        if c == "A":
            layers.append({"type": "latent_attention", "mixer": {"heads": H, "dim": D, "rot_dim": 64, "vdim": D, "kv_rank": 4 * D, "rot": rot,
                                                                 "scale": (D + 64) ** -0.5}, "mlp": mlp})
        else:
            decay = [math.exp(-2.0 ** (-(1 + 7 * h / max(H - 1, 1)))) for h in range(H)]
            layers.append({"type": "lightning", "mixer": {"heads": H, "dim": D, "vdim": D, "decay": decay}, "mlp": mlp})
    return {"architecture": "Nidorax", "layers": layers, "norm": {"eps": 1e-6}, "postln_alpha": 2.0, "vocab": V, "width": W}


def _entry(us: float, flops: float, byts: float, flop_peak: float) -> dict:
    return {"us": round(us, 1), "tflops": round(flops / us / 1e6, 2), "tb_s": round(byts / us / 1e6, 3),
            "of_roofline": round(max(flops / us / 1e6 / flop_peak, byts / us / 1e6 / HBM_TBS), 4)}


def kernel_rooflines(name: str, prompt: int, batch: int, device) -> dict:
    """Each new kernel alone at the size's shapes, beside the like kernel of the post-norm hybrid decoder: microseconds and the
    share of the roofline that bounds it (matrix cores for a prompt portion's attention products, the fp32 vector rate for the
    recurrences, HBM for everything a decode step streams)."""
    from mini_sglang_amd import mixops

    W, order, H, G, D, window, taps, rank, E, top, ff, V = SIZES[name]
    bf = torch.bfloat16
    out = {}

    def rnd(*shape, dtype=bf, scale=1.0):
        return (torch.randn(shape, device=device, dtype=torch.float32) * scale).to(dtype)

    def i32(v):
        return torch.tensor(v, dtype=torch.int32, device=device)

    for phase, T, reqs, ctx in (("prefill", prompt, 1, prompt), ("decode", batch, batch, prompt)):
        q_len = T // reqs
        cu, seq, rows = i32([i * q_len for i in range(reqs + 1)]), i32([ctx] * reqs), i32(list(range(reqs)))
        slots = reqs * ctx
        table = torch.arange(slots, dtype=torch.int32, device=device).view(reqs, ctx)
        # --- windowed attention with mixed heads (+ its like kernel: latent attention at latent 4 D + 64)
        src = rnd(T, H * D + H, scale=0.3)
        kc, vc = rnd(slots, G * D, scale=0.3), rnd(slots, G * D)
        talk = torch.eye(H, device=device) + 0.05 * torch.randn(H, H, device=device)
        o = torch.empty(T, H * D, dtype=bf, device=device)
        wsplits = mixops.window_attn_splits(reqs, T, window, ctx)
        us = _time_us(lambda: mixops.window_attn(o, src, H * D, kc, vc, table, rows, seq, cu, reqs, H, G, D, D, window, D ** -0.5, talk,
                                                 splits=wsplits))
        first = ctx - q_len
        pairs = reqs * sum(min(first + i + 1, window) for i in range(q_len))
        keys_read = reqs * min(ctx, window + q_len - 1)
        out[f"{phase}.window_attn"] = _entry(us, 2.0 * pairs * H * (2 * D + H), keys_read * 2 * G * D * 2 + T * H * D * 4, MFMA_TFLOPS)
        R, r = 4 * D, 64
        cache, q_abs = rnd(slots, R + r), rnd(T, H, R + r, dtype=torch.float32, scale=0.1)
        o_lat = torch.empty(T, H, R, dtype=torch.float32, device=device)
        splits = mixops.latent_attn_splits(reqs, T, H, ctx) if q_len <= 16 else 1
        us = _time_us(lambda: mixops.latent_attn(o_lat, q_abs, cache, table, rows, seq, cu, reqs, R, 0.1, splits=splits))
        pairs_full = reqs * (q_len * first + q_len * (q_len + 1) // 2)
        out[f"{phase}.latent_attn (like)"] = _entry(us, 2.0 * pairs_full * H * (2 * R + r), reqs * ctx * (R + r) * 2 + T * H * (2 * R + r) * 4,
                                                   MFMA_TFLOPS)
        # --- short convolution + unit vectors, delta rule (+ its like kernel: lightning), per-head gated norm
        C = 2 * H * D + H * D
        proj = rnd(T, C + H + H + H * D, scale=0.5)
        tap_w = rnd(C, taps, scale=0.5)
        conv_state = torch.zeros(reqs, taps - 1, C, dtype=bf, device=device)
        us = _time_us(lambda: mixops.short_conv(proj, C, tap_w, conv_state, cu, seq, rows, reqs, 2 * H, H, D))
        out[f"{phase}.short_conv"] = _entry(us, 0.0, T * C * (2 + 4) + reqs * (taps - 1) * C * 4, VALU_TFLOPS)
        qkv = mixops.short_conv(proj, C, tap_w, conv_state, cu, seq, rows, reqs, 2 * H, H, D)
        state = torch.zeros(reqs, H, D, D, dtype=torch.float32, device=device)
        rate = -torch.rand(H, device=device)
        od = torch.empty(T, H * D, dtype=torch.float32, device=device)
        dchunks = None
        if q_len >= 512:  # what the engine's metadata does for long portions: pieces of 256 tokens in parallel
            n = -(-q_len // 256)
            items = i32([[b, c * 256, min((c + 1) * 256, q_len)] for b in range(reqs) for c in range(n)]).view(-1)
            dchunks = (items, i32([b * n for b in range(reqs + 1)]), reqs * n)
        for label, chan in (("delta_rule", False), ("channel_delta_rule", True)):
            a_raw = rnd(T, H * D if chan else H)
            dtb = torch.zeros(H * D if chan else H, dtype=torch.float32, device=device)
            us = _time_us(lambda: mixops.delta_rule(od, qkv, state, proj[:, C: C + H], a_raw, chan, rate, dtb, cu, seq, rows, reqs, H,
                                                    chunks=dchunks))
            byts = 2 * reqs * H * D * D * 4 + T * C * 4 + T * H * D * 4
            out[f"{phase}.{label}"] = _entry(us, 8.0 * T * H * D * D, byts, VALU_TFLOPS)
        lq = rnd(T, 4 * H * D, scale=0.5)
        decay = torch.full((H,), 0.97, dtype=torch.float32, device=device)
        chunks = None
        if q_len >= 256:
            n = -(-q_len // 128)
            items = i32([[b, c * 128, min((c + 1) * 128, q_len)] for b in range(reqs) for c in range(n)]).view(-1)
            chunks = (items, i32([b * n for b in range(reqs + 1)]), reqs * n)
        us = _time_us(lambda: mixops.lightning(od, lq, state, decay, cu, seq, rows, reqs, chunks=chunks))
        out[f"{phase}.lightning (like)"] = _entry(us, 4.0 * T * H * D * D, 2 * reqs * H * D * D * 4 + T * 3 * H * D * 2 + T * H * D * 4, VALU_TFLOPS)
        gate, nw = rnd(T, H * D), rnd(D, scale=0.1)
        us = _time_us(lambda: mixops.head_gated_norm(od, gate, nw, 1e-6, H, D, mixops.GATE_SILU))
        out[f"{phase}.head_gated_norm"] = _entry(us, 0.0, T * H * D * (4 + 2 + 2), VALU_TFLOPS)
        # --- residual sum + depth average over 4 stored rows + norm (+ router); like kernel: the post-norm
        hist = rnd(5, T, W, dtype=torch.float32)
        depth_w = torch.full((5,), 0.2, dtype=torch.float32, device=device)
        x, y, nw2 = rnd(T, W, dtype=torch.float32), rnd(T, W), rnd(W, scale=0.1)
        x_out, h_out = torch.empty_like(x), torch.empty(T, W, dtype=bf, device=device)
        us = _time_us(lambda: mixops.prenorm(x, y=y, sum_out=hist[4], history=hist, depth_w=depth_w, x_out=x_out, weight=nw2, h_out=h_out))
        out[f"{phase}.prenorm_depth5"] = _entry(us, 0.0, T * W * (4 + 2 + 4 + 4 * 4 + 4 + 2), VALU_TFLOPS)
        router, bias = rnd(E, W, scale=W ** -0.5), rnd(E, scale=0.01)
        us = _time_us(lambda: mixops.prenorm(x, y=y, sum_out=x_out, weight=nw2, h_out=h_out, route=(router, bias, top)))
        out[f"{phase}.prenorm_route"] = _entry(us, 0.0, T * W * (4 + 2 + 4 + 2) + E * W * 2, VALU_TFLOPS)
        us = _time_us(lambda: mixops.postnorm(x, nw2, 1e-6, y=y, alpha=2.0, x_out=x_out, h_out=h_out))
        out[f"{phase}.postnorm (like)"] = _entry(us, 0.0, T * W * (4 + 2 + 4 + 2), VALU_TFLOPS)
        # --- feed-forwards: polynomial activation, gated experts (gate | up product, SiLU x up, down product)
        z = rnd(T, top * ff)
        coef = torch.tensor([1.0, 0.3, 0.1, 0.0], dtype=torch.float32, device=device)
        us = _time_us(lambda: mixops.poly_act(z, coef, 1e-6))
        out[f"{phase}.poly_act"] = _entry(us, 0.0, T * top * ff * 6, VALU_TFLOPS)  # the row is read twice: once from HBM, once from L2
        h = rnd(T, W)
        ids, _ = mixops.route_top(h, router, bias, top)
        seg, perm = mixops.moe_sort(ids, E)
        n = T * top
        up, down = rnd(E, 2 * ff, W, scale=W ** -0.5), rnd(E, W, ff, scale=ff ** -0.5)
        gu, yv = torch.empty(n, 2 * ff, dtype=bf, device=device), torch.empty(T, top, W, dtype=bf, device=device)
        us_u = _time_us(lambda: mixops.gemm_nt(gu, h, up, n, 2 * ff, W, lda=W, ldb=W, ldc=2 * ff, groups=E, b_gs=2 * ff * W, seg=seg,
                                               a_rows=perm, a_div=top))
        us_a = _time_us(lambda: mixops.silu_mul(gu))
        act = mixops.silu_mul(gu)
        us_d = _time_us(lambda: mixops.gemm_nt(yv, act, down, n, W, ff, lda=ff, ldb=ff, ldc=W, groups=E, b_gs=W * ff, seg=seg, c_rows=perm))
        touched = min(E, n)
        out[f"{phase}.experts_gate_up"] = _entry(us_u, 4.0 * n * ff * W, touched * 2 * ff * W * 2 + n * (W + 2 * ff) * 2, MFMA_TFLOPS)
        out[f"{phase}.silu_mul"] = _entry(us_a, 0.0, n * ff * 6, VALU_TFLOPS)
        out[f"{phase}.experts_down"] = _entry(us_d, 2.0 * n * ff * W, touched * ff * W * 2 + n * (W + ff) * 2, MFMA_TFLOPS)
    return out


def main(argv=None) -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", nargs="*", default=["s", "m"], choices=sorted(SIZES))
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-twin", action="store_true", help="skip the post-norm hybrid decoder of equal size")
    ap.add_argument("--no-kernels", action="store_true")
    args = ap.parse_args(argv)
    from mini_sglang_amd.hybrid import HybridConfig, bedarax_config

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    report = {"metric": "bedarax_decoder_throughput", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
              "prompt": args.prompt, "batch": args.batch, "steps": args.steps, "sizes": {}}
    keys = ("width", "layers", "heads", "kv_heads", "head", "window", "taps", "rank", "experts", "top", "ff", "vocab")
    for name in args.sizes:
        entry = {"shape": dict(zip(keys, SIZES[name]))}
        entry["bedarax"] = run_engine(bedarax_config(bedarax_json(name), bedarax_shapes(name)), args.prompt, args.batch, args.steps,
                                      args.warmup, device)
        print(f"[bedarax bench] {name}: " + json.dumps(entry["bedarax"]), flush=True)
        if not args.no_twin:
            entry["post_norm_hybrid"] = run_engine(HybridConfig.from_json(twin_json(name)), args.prompt, args.batch, args.steps, args.warmup,
                                                   device)
            print(f"[bedarax bench] {name} twin: " + json.dumps(entry["post_norm_hybrid"]), flush=True)
        if not args.no_kernels:
            entry["kernels"] = kernel_rooflines(name, args.prompt, args.batch, device)
        report["sizes"][name] = entry
    print(json.dumps(report))


if __name__ == "__main__":
    main()
