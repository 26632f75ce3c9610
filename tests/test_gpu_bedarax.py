"""The pre-norm hybrid decoder (Bedarax: windowed attention with mixed heads, gated delta-rule layers, depth-averaged
stream, polynomial and gated-expert feed-forwards) on the GPU against the plain restatement in tests/bedarax_oracle.py:
small configurations and random weights made here, the engine's own step function, cache, state slots and kernels on one
side, whole-sequence float64 arithmetic on the other.

fp32 engines are held to 2e-4 of the largest reference value (the sharp test); bf16 engines to the rounding of a 16-bit
product chain.  Where random weights would hide a fault the inputs are built so that it shows: one key whose score
stands out just inside or just outside the window, a state slot that still holds its last owner's state.
"""
from __future__ import annotations

import json
import math

import pytest
import torch

import bedarax_oracle as O
from test_gpu_hybrid import alone, rel, replay, tokens_of

pytestmark = pytest.mark.gpu

FP32_TOL = 2e-4
BF16_TOL = 6e-2


# ----------------------------------------------------------------------------------------- configurations
def moe(experts=6, top=2, ff=40):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def att(heads=4, kv_heads=2, dim=24, vdim=40, window=20, scale=0.3, v_mix=False, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m, "mlp": mlp}


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, mlp=None, channel=False):
    return {"type": "channel_delta" if channel else "delta",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def config(layers, width=48, vocab=80, eps=1e-5):
    return {"architecture": "Bedarax", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


FULL = config([delta(mlp=moe()), att(v_mix=True, mlp=dense()), delta(channel=True, heads=3, kv_heads=3, dim=8, vdim=16, conv=4, mlp=None),
               att(heads=2, kv_heads=2, dim=12, vdim=40, window=33, v_mix=True, mlp=moe(experts=4, top=1, ff=24)),
               delta(channel=True, heads=4, kv_heads=1, dim=12, vdim=8, conv=2, mlp=moe(experts=5, top=5, ff=16))])


# ----------------------------------------------------------------------------------------- harness
_ENGINES: dict = {}


def engine_for(cfg_json, dtype, max_tokens=512, rows=4, page_size=16, graphs=None, seed=5):
    """(engine, checkpoint-named weights on the host) for a configuration; engines are kept for the session."""
    from mini_sglang_amd.engine import Engine, EngineConfig
    from mini_sglang_amd.hybrid import bedarax_config

    key = (json.dumps(cfg_json, sort_keys=True), dtype, max_tokens, rows, page_size, tuple(graphs or ()), seed)
    if key not in _ENGINES:
        pages = max_tokens // page_size
        eng = Engine(EngineConfig(model=bedarax_config(cfg_json), dtype=dtype, max_running_req=rows, page_size=page_size,
                                  num_page_override=pages, max_seq_len_override=pages * page_size, cuda_graph_bs=list(graphs or []),
                                  gemm_tune="off", refine_in_graph=False, seed=seed), torch.device("cuda:0"))
        _ENGINES[key] = (eng, eng.model.export_state())
    return _ENGINES[key]


def check(eng_state, cfg_json, steps, seqs, tol, allow=0.0):
    """Every position of every request within `tol` of the restatement; `allow` = the share of positions that may miss it
    (16-bit runs only: a router choice that rests on a close call flips under rounding and moves that token's logits)."""
    eng, state = eng_state
    got = replay(eng, steps)
    for rid, toks in seqs.items():
        ref = O.forward(cfg_json, state, toks)
        assert got[rid].shape == ref.shape
        per = (got[rid] - ref).abs().amax(1) / ref.abs().max()
        bad = (per > tol).nonzero().flatten().tolist()
        assert len(bad) <= allow * len(toks), f"request {rid}: {len(bad)} of {len(toks)} positions above {tol} " \
                                              f"(worst {float(per.max()):.3e}, first at {bad[0]})"
    return got


# ----------------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("layer", [
    att(), att(heads=3, kv_heads=3, dim=10, vdim=6, window=7), att(heads=6, kv_heads=1, dim=8, vdim=72, window=0),
    att(heads=1, kv_heads=1, dim=40, vdim=8, window=1), att(heads=5, kv_heads=5, dim=16, vdim=16, window=64, scale=1.0),
    delta(), delta(heads=3, kv_heads=3, dim=20, vdim=70, conv=4), delta(heads=2, kv_heads=1, dim=40, vdim=12, conv=1),
    delta(heads=1, kv_heads=1, dim=72, vdim=8, conv=6),
    delta(channel=True), delta(channel=True, heads=2, kv_heads=2, dim=36, vdim=80, conv=5),
    delta(heads=2, kv_heads=1, dim=64, vdim=16), delta(channel=True, heads=1, kv_heads=1, dim=128, vdim=72, conv=2),
    delta(heads=1, kv_heads=1, dim=192, vdim=8, conv=2),
], ids=["attention-grouped", "attention-odd-sizes", "attention-no-window", "attention-window-one", "attention-window-at-tile",
        "delta-grouped", "delta-wide-v", "delta-one-tap", "delta-wide-key", "channel-delta-grouped", "channel-delta-wide",
        "delta-key-64", "channel-delta-key-128", "delta-key-192"])
def test_mixer_alone_fp32(layer):
    cfg = config([layer])
    toks = tokens_of(70, cfg["vocab"], 1)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [70]), {"a": toks}, FP32_TOL)


def test_attention_many_wide_heads_bf16():
    """Twelve heads of 128: the 8-token query tile needs more LDS than a kernel gets by default; 16-bit keys and values."""
    cfg = config([att(heads=12, kv_heads=4, dim=128, vdim=32, window=40, scale=0.09)], width=64)
    toks = tokens_of(150, cfg["vocab"], 12)
    check(engine_for(cfg, torch.bfloat16), cfg, alone("a", toks, [100, 1, 1, 5, 43]), {"a": toks}, BF16_TOL)


@pytest.mark.parametrize("mlp", [dense(), dense(ff=300), moe(), moe(experts=4, top=1), moe(experts=3, top=3, ff=8), moe(experts=70, top=6, ff=16)],
                         ids=["dense", "dense-wide", "experts", "top-1", "all-experts", "many-experts"])
def test_feed_forward_alone_fp32(mlp):
    cfg = config([delta(heads=1, kv_heads=1, dim=4, vdim=4, conv=2, mlp=mlp)])
    toks = tokens_of(50, cfg["vocab"], 2)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [50]), {"a": toks}, FP32_TOL)


def test_value_mixing_across_layers_fp32():
    """Three value-mixing layers with an unmixed one between them: the second and third blend with the FIRST one's values."""
    cfg = config([att(v_mix=True), att(v_mix=False, heads=2, kv_heads=1, vdim=16), att(v_mix=True, heads=2, dim=8, window=0), att(v_mix=True)])
    toks = tokens_of(60, cfg["vocab"], 11)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [31, 1, 28]), {"a": toks}, FP32_TOL)


def test_layer_outputs_fp32():
    """The residual stream after every layer (after its depth average), not only the logits."""
    eng, state = engine_for(FULL, torch.float32)
    toks = tokens_of(40, FULL["vocab"], 3)
    mine: list = []
    orig = eng.model.forward
    eng.model.forward = lambda ctx, b, logits_out=None: orig(ctx, b, logits_out, layer_outputs=mine)
    try:
        replay(eng, alone("a", toks, [40]))
    finally:
        eng.model.forward = orig
    ref: list = []
    O.forward(FULL, state, toks, layer_outputs=ref)
    assert len(mine) == len(ref) == len(FULL["layers"])
    for i, (a, b) in enumerate(zip(mine, ref)):
        assert rel(a.double().cpu(), b) < FP32_TOL, f"layer {i}"


# ----------------------------------------------------------------------------------------- kernels on built inputs
def _window_reference(q, k, v, gate, talk, scale, window, rep):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of ONE sequence in float64 -> [T, H, dv]."""
    T = q.shape[0]
    raw = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1)) * scale
    s = torch.einsum("hg,gij->hij", talk, raw)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (j <= i) & ((i - j < window) if window else (j <= i))
    p = torch.softmax(s.masked_fill(~seen[None], -math.inf), -1)
    return torch.einsum("hij,jhe->ihe", p, v.repeat_interleave(rep, 1)) * torch.sigmoid(gate)[:, :, None]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("splits", [1, 3], ids=["one-range", "three-ranges"])
@pytest.mark.parametrize("window", [1, 5, 16, 17, 63, 64, 65, 130, 0])
def test_window_edges_one_key_stands_out(dev, dtype, window, splits):
    """One loud key: every query that still sees it must put (nearly) all its weight there, the first query past the window
    none.  The sequence is cut into a prompt portion and single decoded tokens, its slots are scattered over the pool, and the
    loud key sits so that its last visible query falls once in the portion and once among the decoded tokens; with the keys
    of every token in one range and cut into three (partial results merged)."""
    from mini_sglang_amd import mixops

    H, G, d, dv, scale = 4, 2, 16, 24, 0.5
    T = 200
    for loud, cut in ((3, 150), (100, 150), (30, 40), (149, 150), (0, 1)):
        g = torch.Generator().manual_seed(window * 1000 + loud)
        q = torch.randn(T, H, d, generator=g, dtype=torch.float64) * 0.3
        k = torch.randn(T, G, d, generator=g, dtype=torch.float64) * 0.3
        v = torch.randn(T, G, dv, generator=g, dtype=torch.float64)
        gate = torch.randn(T, H, generator=g, dtype=torch.float64)
        talk = torch.eye(H, dtype=torch.float64) + 0.1 * torch.randn(H, H, generator=g, dtype=torch.float64)
        k[loud] = 0.0
        k[loud, :, 0] = 12.0
        q[:, :, 0] = 4.0  # raw score of the loud key: 48 * scale for every head
        q, k, v, gate = (t.to(dtype).double() for t in (q, k, v, gate))
        ref = _window_reference(q, k, v, gate, talk.float().double(), scale, window, H // G)
        slots = torch.randperm(512, generator=g)[:T].to(torch.int32)
        table = torch.zeros((3, 256), dtype=torch.int32)
        table[2, :T] = slots
        kc = torch.zeros((512, G * d), dtype=dtype, device=dev)
        vc = torch.zeros((512, G * dv), dtype=dtype, device=dev)
        kc[slots.long().to(dev)] = k.reshape(T, -1).to(dtype).to(dev)
        vc[slots.long().to(dev)] = v.reshape(T, -1).to(dtype).to(dev)
        src = torch.cat([q.reshape(T, -1), gate], 1).to(dtype).to(dev)
        got = torch.empty((T, H * dv), dtype=dtype, device=dev)
        # a portion of request row 2 up to `cut`, then 70 tokens alone, then the rest as a second portion
        single_end = min(T, cut + 70)
        pieces = [(0, cut)] + [(t, t + 1) for t in range(cut, single_end)] + ([(single_end, T)] if single_end < T else [])
        for lo, hi in pieces:
            part = torch.empty((hi - lo, H * dv), dtype=dtype, device=dev)
            mixops.window_attn(part, src[lo:hi], H * d, kc, vc, table.to(dev), torch.tensor([2], dtype=torch.int32, device=dev),
                               torch.tensor([hi], dtype=torch.int32, device=dev), torch.tensor([0, hi - lo], dtype=torch.int32, device=dev),
                               1, H, G, d, dv, window, scale, talk.float().to(dev), splits=splits)
            got[lo:hi] = part
        got = got.double().cpu().view(T, H, dv)
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert float((got - ref).abs().max()) < tol * float(ref.abs().max()), (window, loud, cut)
        if window:  # the edge itself: last query inside, first query outside
            inside, outside = loud + window - 1, loud + window
            if inside < T and window > 1:
                want = v[loud].repeat_interleave(H // G, 0) * torch.sigmoid(gate[inside])[:, None]
                assert float((got[inside] - want).abs().max()) < 2e-2 * float(want.abs().max()) + 1e-3
            if outside < T:
                want = v[loud].repeat_interleave(H // G, 0) * torch.sigmoid(gate[outside])[:, None]
                assert float((got[outside] - want).abs().max()) > 0.05 * float(want.abs().max())


@pytest.mark.parametrize("chunk", [0, 1, 5], ids=["whole", "chunks-of-1", "chunks-of-5"])
def test_delta_rule_state_slots_and_cuts(dev, chunk):
    """The recurrence kernel alone: two requests in one launch on state rows that hold garbage, then continued in a second
    launch; per-head and per-channel decays, grouped keys; whole portions, and portions cut into pieces that run in parallel
    and are joined by the scan.  Against the token loop of the restatement."""
    from mini_sglang_amd import mixops

    for per_channel in (False, True):
        H, G, d, dv = 4, 2, 12, 20
        g = torch.Generator().manual_seed(7 + per_channel)
        lens = [23, 9]
        seq = {}
        for b, n in enumerate(lens):
            qk = torch.randn(n, 2 * G, d, generator=g, dtype=torch.float64)
            qk = qk / qk.norm(dim=-1, keepdim=True)
            seq[b] = dict(q=qk[:, :G] * d ** -0.5, k=qk[:, G:], v=torch.randn(n, H, dv, generator=g, dtype=torch.float64),
                          b=torch.randn(n, H, generator=g, dtype=torch.float64),
                          a=torch.randn(n, H * d if per_channel else H, generator=g, dtype=torch.float64))
        rate = -torch.exp(torch.randn(H, generator=g, dtype=torch.float64) * 0.5)
        dtb = torch.randn(H * d if per_channel else H, generator=g, dtype=torch.float64) * 0.5
        state = torch.randn((3, H, d, dv), generator=g, dtype=torch.float32).to(dev)  # garbage: a fresh request must not read it
        outs = {b: [] for b in seq}
        for lo, hi in ((0.0, 0.6), (0.6, 1.0)):
            cuts = {b: (int(lo * n), int(hi * n)) for b, n in enumerate(lens)}
            rows = [torch.cat([seq[b]["q"][s:e].reshape(e - s, -1), seq[b]["k"][s:e].reshape(e - s, -1), seq[b]["v"][s:e].reshape(e - s, -1)], 1)
                    for b, (s, e) in cuts.items()]
            qkv = torch.cat(rows).float().to(dev)
            b_raw = torch.cat([seq[b]["b"][s:e] for b, (s, e) in cuts.items()]).float().to(dev)
            a_raw = torch.cat([seq[b]["a"][s:e] for b, (s, e) in cuts.items()]).float().to(dev)
            cu = torch.tensor([0, cuts[0][1] - cuts[0][0], qkv.shape[0]], dtype=torch.int32, device=dev)
            out = torch.empty((qkv.shape[0], H * dv), dtype=torch.float32, device=dev)
            chunks = None
            if chunk:
                items, firsts = [], [0]
                for bb, (s0, e0) in cuts.items():
                    items += [[bb, c, min(c + chunk, e0 - s0)] for c in range(0, e0 - s0, chunk)]
                    firsts.append(len(items))
                chunks = (torch.tensor(items, dtype=torch.int32, device=dev).view(-1), torch.tensor(firsts, dtype=torch.int32, device=dev),
                          len(items))
            mixops.delta_rule(out, qkv, state, b_raw, a_raw, per_channel, rate.float().to(dev), dtb.float().to(dev), cu,
                              torch.tensor([cuts[0][1], cuts[1][1]], dtype=torch.int32, device=dev),
                              torch.tensor([2, 0], dtype=torch.int32, device=dev), 2, G, chunks=chunks)
            outs[0].append(out[: cu[1]].cpu())
            outs[1].append(out[cu[1]:].cpu())
        for b, n in enumerate(lens):
            s = seq[b]
            a = s["a"] + dtb
            decay = torch.exp(rate[None, :, None] * torch.nn.functional.softplus(a.view(n, H, d))) if per_channel else \
                torch.exp(rate[None, :] * torch.nn.functional.softplus(a))
            ref = O.delta_rule(s["q"].repeat_interleave(H // G, 1), s["k"].repeat_interleave(H // G, 1), s["v"], torch.sigmoid(s["b"]), decay)
            got = torch.cat(outs[b]).double().view(n, H, dv)
            assert rel(got, ref) < 1e-5, (per_channel, b)


# ----------------------------------------------------------------------------------------- schedules
@pytest.mark.parametrize("dtype,tol", [(torch.float32, FP32_TOL), (torch.bfloat16, BF16_TOL)], ids=["fp32", "bf16"])
def test_whole_prompt(dtype, tol):
    toks = tokens_of(150, FULL["vocab"], 4)
    check(engine_for(FULL, dtype), FULL, alone("a", toks, [150]), {"a": toks}, tol, allow=0.0 if dtype == torch.float32 else 0.1)


def test_prefill_against_token_by_token_fp32():
    eng_state = engine_for(FULL, torch.float32)
    toks = tokens_of(90, FULL["vocab"], 5)
    whole = check(eng_state, FULL, alone("a", toks, [90]), {"a": toks}, FP32_TOL)["a"]
    single = check(eng_state, FULL, alone("a", toks, [1]), {"a": toks}, FP32_TOL)["a"]
    assert rel(single, whole) < 2e-5


@pytest.mark.parametrize("sizes", [[2], [3, 2, 5], [16], [15, 17], [64, 1, 63, 2], [33, 1, 1, 1, 7], [1, 2, 1, 3]])
def test_portions_fp32(sizes):
    """Portions shorter than the convolutions' reach (2, 1 and 3 tokens against up to 4 taps), at page and window edges."""
    eng_state = engine_for(FULL, torch.float32)
    toks = tokens_of(131, FULL["vocab"], 6)
    check(eng_state, FULL, alone("a", toks, sizes), {"a": toks}, FP32_TOL)


def test_long_portions_run_as_parallel_chunks_fp32():
    """Portions long enough for the delta-rule layers to cut them into pieces (states joined by a scan): first a long portion
    from position 0, then a single token, then a long portion that continues from a carried state, beside a short request;
    lengths off the piece size."""
    eng_state = engine_for(FULL, torch.float32, max_tokens=2048)
    a, b = tokens_of(1200, FULL["vocab"], 30), tokens_of(6, FULL["vocab"], 31)
    steps = [[("a", a[:560], False)], [("a", a[560:561], False), ("b", b[:5], False)], [("b", b[5:], True), ("a", a[561:], True)]]
    got = check(eng_state, FULL, steps, {"a": a, "b": b}, FP32_TOL)
    whole = replay(eng_state[0], alone("a", a, [257, 443]))["a"]
    assert rel(got["a"], whole) < 2e-5


def test_long_decoding_fp32():
    """A short prompt, then 260 tokens one by one: the windows pass over decoded tokens only, the states carry the rest."""
    cfg = config([delta(mlp=moe()), att(window=50, mlp=None), delta(channel=True, heads=2, kv_heads=2, dim=12, vdim=20), att(window=0)])
    toks = tokens_of(270, cfg["vocab"], 7)
    steps = [[("a", toks[:10], False)]] + [[("a", [t], j == 259)] for j, t in enumerate(toks[10:])]
    check(engine_for(cfg, torch.float32), cfg, steps, {"a": toks}, FP32_TOL)


def test_first_tokens_fp32():
    """Positions 0, 1, 2 of a sequence: a one-token request, and requests whose first portion is one or two tokens."""
    eng_state = engine_for(FULL, torch.float32)
    one = tokens_of(1, FULL["vocab"], 8)
    check(eng_state, FULL, alone("a", one, [1]), {"a": one}, FP32_TOL)
    toks = tokens_of(20, FULL["vocab"], 9)
    check(eng_state, FULL, alone("a", toks, [1, 2, 17]), {"a": toks}, FP32_TOL)
    check(eng_state, FULL, alone("a", toks, [2, 1, 17]), {"a": toks}, FP32_TOL)


def test_mixed_batches_against_each_alone_fp32():
    """Four unequal requests: portions of some beside single tokens of others, requests that sit out steps and that end
    while others go on.  Every request must come out as it does alone."""
    eng_state = engine_for(FULL, torch.float32, max_tokens=512)
    seqs = {i: tokens_of(n, FULL["vocab"], 20 + k) for k, (i, n) in enumerate([("a", 97), ("b", 40), ("c", 5), ("d", 130)])}
    at = {i: 0 for i in seqs}
    plan = [{"a": 30, "b": 1, "d": 64}, {"a": 1, "b": 17, "c": 2}, {"d": 2, "a": 1}, {"a": 33, "b": 1, "c": 3, "d": 1},
            {"b": 21, "d": 63}, {"a": 32}]
    steps = []
    for p in plan:
        step = []
        for i, c in p.items():
            t = seqs[i][at[i]: at[i] + c]
            at[i] += len(t)
            step.append((i, t, at[i] == len(seqs[i])))
        steps.append(step)
    assert all(at[i] == len(seqs[i]) for i in seqs)
    mixed = check(eng_state, FULL, steps, seqs, FP32_TOL)
    for i, toks in seqs.items():
        solo = replay(eng_state[0], alone(i, toks, [len(toks)]))[i]
        assert rel(mixed[i], solo) < 2e-5, i


def test_pages_and_state_slots_used_again_fp32():
    """A pool of 8 pages and two request rows: every request after the first runs on pages and on state slots (recurrent
    state AND convolution inputs) that still hold another request's; a request that ends frees them for the next one."""
    cfg = config([delta(conv=4), att(window=25), delta(channel=True, heads=2, kv_heads=2, dim=8, vdim=8, conv=3, mlp=moe())])
    eng_state = engine_for(cfg, torch.float32, max_tokens=128, rows=2)
    seqs = {i: tokens_of(n, cfg["vocab"], 40 + k) for k, (i, n) in enumerate([("a", 60), ("b", 64), ("c", 50), ("d", 33), ("e", 64)])}
    steps = [[("a", seqs["a"][:40], False), ("b", seqs["b"][:30], False)],
             [("a", seqs["a"][40:], True), ("b", seqs["b"][30:], True)],
             [("c", seqs["c"][:2], False)],
             [("c", seqs["c"][2:], True), ("d", seqs["d"][:1], False)],
             [("d", seqs["d"][1:], True)],
             [("e", seqs["e"], True)]]
    check(eng_state, cfg, steps, seqs, FP32_TOL)


def test_other_orders_and_sizes_bf16():
    """Another order of layers, widths that are not powers of two, one expert per token, no feed-forward in a layer: the
    16-bit path end to end."""
    cfg = config([att(heads=2, kv_heads=2, dim=12, vdim=20, window=40, v_mix=True, mlp=moe(experts=3, top=1, ff=20)),
                  delta(channel=True, heads=3, kv_heads=1, dim=12, vdim=28, conv=2, mlp=dense(ff=90)),
                  att(heads=4, kv_heads=2, dim=12, vdim=20, window=0, v_mix=True), delta(heads=3, kv_heads=3, dim=12, vdim=28, mlp=moe())],
                 width=72, vocab=101, eps=1e-6)
    toks = tokens_of(120, cfg["vocab"], 10)
    check(engine_for(cfg, torch.bfloat16), cfg, alone("a", toks, [50, 1, 1, 30, 2, 36]), {"a": toks}, BF16_TOL, allow=0.1)


# ----------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("graphs", [None, [1, 2, 4]], ids=["eager", "graphs"])
def test_greedy_generation_through_the_scheduler(graphs):
    """OfflineRunner.generate (chunked prefill with a small budget, continuous decode, the sampler's argmax, captured
    decode graphs) against greedy decoding with the restatement; a step whose two best logits are closer than the fp32
    tolerance ends the comparison for that request."""
    from mini_sglang_amd.core import SamplingParams
    from mini_sglang_amd.offline import OfflineRunner

    eng, state = engine_for(FULL, torch.float32, max_tokens=512, graphs=graphs)
    prompts = [tokens_of(n, FULL["vocab"], 60 + n) for n in (9, 31, 47)]
    run = OfflineRunner(eng, max_extend_tokens=32, seed=2)
    n_new = 12
    run.generate(prompts, [SamplingParams(temperature=0.0, max_tokens=n_new, ignore_eos=True)] * len(prompts))
    compared = 0
    for p, st in zip(prompts, run.last_states):
        out = run.output_ids(st)
        assert len(out) == n_new
        seq = list(p)
        for tok in out:
            lg = O.forward(FULL, state, seq)[-1]
            top2 = lg.topk(2).values
            if float(top2[0] - top2[1]) < 1e-3 * float(lg.abs().max()):
                break
            assert tok == int(lg.argmax()), (len(seq), tok)
            seq.append(tok)
            compared += 1
    assert compared >= 2 * n_new


def test_trace_command_line(tmp_path):
    """bin/trace_run end to end in its own process on a checkpoint folder written here: the model class comes from
    config.json, the inner sizes of the two-step projections from the checkpoint's tensor shapes."""
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np
    from safetensors.torch import save_file

    from mini_sglang_amd.hybrid import HybridDecoder, bedarax_config

    cfg = config([att(heads=3, kv_heads=1, dim=10, vdim=14, window=12, v_mix=True, mlp=moe(experts=6, top=2, ff=26)),
                  delta(channel=True, heads=3, kv_heads=3, dim=10, vdim=18, conv=3, mlp=dense(ff=44)),
                  att(heads=2, kv_heads=1, dim=10, vdim=14, window=0, v_mix=True)], width=100, vocab=131)
    shapes = {"l1.mix.a1": (7, 100), "l1.mix.g1": (9, 100)}
    model = HybridDecoder(bedarax_config(cfg, shapes), dtype=torch.bfloat16, device=torch.device("cpu"), seed=9)
    state = model.export_state()
    assert state["l1.mix.a2"].shape == (30, 7) and state["l1.mix.g2"].shape == (54, 9)
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    (mdir / "config.json").write_text(json.dumps(cfg))
    save_file(state, str(mdir / "model.safetensors"))
    a, b = tokens_of(45, cfg["vocab"], 70), tokens_of(9, cfg["vocab"], 71)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}, {"id": "a", "tokens": a[30:31], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[31:], "want": [13]}, {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]}]
    root = Path(__file__).resolve().parent.parent
    pr = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(mdir), "--dtype", "float32", "--out", str(out),
                         "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True, capture_output=True,
                        timeout=110)
    assert pr.returncode == 0, pr.stderr[-2000:]
    assert [ln for ln in pr.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    ra, rb = O.forward(cfg, state, a), O.forward(cfg, state, b)
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1)).double()
    got1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(1, -1)).double()
    got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)).double()
    assert rel(got0, ra[[0, 29]]) < FP32_TOL and rel(got1, ra[[30]]) < FP32_TOL
    assert rel(got2, torch.stack([ra[44], rb[8]])) < FP32_TOL
    # the same folder through `generate`: greedy tokens in 16 bits, in range and of the asked length
    pr = subprocess.run([sys.executable, "-m", "mini_sglang_amd.cli", "generate", "--model", str(mdir), "--prompt", "5,17,3", "--prompt",
                         ",".join(map(str, a[:20])), "--max-tokens", "6"], cwd=str(root), text=True, capture_output=True, timeout=110)
    assert pr.returncode == 0, pr.stderr[-2000:]
    outs = [json.loads(ln)["output"] for ln in pr.stdout.splitlines() if ln.startswith("{")]
    assert len(outs) == 2 and all(len(o) == 6 and all(0 <= t < cfg["vocab"] for t in o) for o in outs)
