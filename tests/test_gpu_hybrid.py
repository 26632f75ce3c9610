"""The hybrid decoder (latent attention + lightning recurrence + routed experts) on the GPU against the plain
restatement in tests/hybrid_oracle.py: small configurations and random weights made here, the engine's own step function,
cache, state slots and kernels on one side, whole-sequence float64 arithmetic on the other.

fp32 engines are held to 2e-4 of the largest reference value (the sharp test); bf16 engines to the rounding of a
16-bit product chain.  Where random weights would hide a fault the inputs are built so that it shows (one far key that
takes all the attention, choice scores that are all negative, a state slot that still holds its last owner's state).
"""
from __future__ import annotations

import math

import pytest
import torch

import hybrid_oracle as O

pytestmark = pytest.mark.gpu

FP32_TOL = 2e-4
BF16_TOL = 6e-2


# ----------------------------------------------------------------------------------------- configurations
def moe(experts=6, top=2, ff=40, count=3, keep=2):
    r = {"experts": experts, "top": top}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r}


def lat(heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=48, kv_from=None, dims=None, scaling=True, base=5000.0, mlp=None):
    rot = {"base": base, "dims": dims or rot_dim}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "fast": 16.0, "original": 64, "slow": 2.0}
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot,
         "scale": 1.0 / math.sqrt(dim + rot_dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def lit(heads=4, dim=8, vdim=24, decay=None, mlp=None):
    decay = decay or [0.5 + 0.499 * i / max(heads - 1, 1) for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp}


def config(layers, width=48, vocab=80, alpha=1.7, eps=1e-5):
    return {"architecture": "Nidorax", "layers": layers, "norm": {"eps": eps}, "postln_alpha": alpha, "vocab": vocab, "width": width}


FULL = config([lit(mlp=moe()), lat(mlp=moe(experts=4, top=1, ff=24, count=0)), lit(heads=2, dim=16, vdim=8, mlp=None),
               lat(kv_from=1, heads=5, dim=8, vdim=16, mlp=moe(experts=8, top=3, ff=16, count=4, keep=3))])


# ----------------------------------------------------------------------------------------- harness
_ENGINES: dict = {}


def engine_for(cfg_json, dtype, max_tokens=512, rows=4, page_size=16, graphs=None, seed=5):
    """(engine, checkpoint-named weights on the host) for a configuration; engines are kept for the session."""
    import json

    from mini_sglang_amd.engine import Engine, EngineConfig
    from mini_sglang_amd.hybrid import HybridConfig

    key = (json.dumps(cfg_json, sort_keys=True), dtype, max_tokens, rows, page_size, tuple(graphs or ()), seed)
    if key not in _ENGINES:
        pages = max_tokens // page_size
        eng = Engine(EngineConfig(model=HybridConfig.from_json(cfg_json), dtype=dtype, max_running_req=rows, page_size=page_size,
                                  num_page_override=pages, max_seq_len_override=pages * page_size, cuda_graph_bs=list(graphs or []),
                                  gemm_tune="off", refine_in_graph=False, seed=seed), torch.device("cuda:0"))
        _ENGINES[key] = (eng, eng.model.export_state())
    return _ENGINES[key]


def tokens_of(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, steps):
    """steps: list of lists of (request id, tokens, last?) -> {id: logits [its tokens, vocab] float64 on the host}; every
    position is asked for."""
    from mini_sglang_amd.offline import StepReplayer

    rep = StepReplayer(eng, seed=1)
    got: dict = {}
    for step in steps:
        entries = [{"id": i, "tokens": t, "want": list(range(len(t)))} for i, t, _ in step]
        lg = rep.step(entries, [i for i, _, last in step if last])
        at = 0
        for i, t, _ in step:
            got.setdefault(i, []).append(lg[at: at + len(t)].double().cpu())
            at += len(t)
    assert not rep.live
    return {i: torch.cat(v) for i, v in got.items()}


def portions(tokens, sizes):
    out, at, k = [], 0, 0
    while at < len(tokens):
        c = min(sizes[k % len(sizes)], len(tokens) - at)
        out.append(tokens[at: at + c])
        at, k = at + c, k + 1
    return out


def alone(rid, tokens, sizes):
    p = portions(tokens, sizes)
    return [[(rid, t, j == len(p) - 1)] for j, t in enumerate(p)]


def rel(got, ref):
    return float((got - ref).abs().max() / ref.abs().max())


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
    lit(), lit(heads=1, dim=20, vdim=72), lit(heads=3, dim=40, vdim=12, decay=[1.0, 0.999, 0.1]),
    lat(), lat(heads=1, dim=8, rot_dim=16, vdim=8, kv_rank=24), lat(dims=4), lat(scaling=False), lat(heads=18, dim=8, vdim=8, kv_rank=16),
], ids=["lightning", "lightning-wide-v", "lightning-decays", "latent", "latent-one-head", "latent-partial-rotation",
        "latent-unscaled", "latent-many-heads"])
def test_mixer_alone_fp32(layer):
    cfg = config([layer])
    toks = tokens_of(70, cfg["vocab"], 1)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [70]), {"a": toks}, FP32_TOL)


@pytest.mark.parametrize("mlp", [moe(), moe(experts=4, top=1, count=0), moe(experts=8, top=4, ff=8, count=2, keep=1),
                                 moe(experts=9, top=3, ff=56, count=3, keep=3)],
                         ids=["grouped", "top1-no-groups", "one-group-kept", "all-groups-kept"])
def test_feed_forward_alone_fp32(mlp):
    cfg = config([lit(heads=1, dim=4, vdim=4, mlp=mlp)])
    toks = tokens_of(50, cfg["vocab"], 2)
    check(engine_for(cfg, torch.float32), cfg, alone("a", toks, [50]), {"a": toks}, FP32_TOL)


def test_layer_outputs_fp32():
    """The residual stream after every layer, not only the logits."""
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


def test_router_negative_choices_and_groups(dev):
    """All choice scores negative (large negative corrections): an expert outside the kept groups must lose to every expert
    inside them (minus infinity, not zero), and the weights are the uncorrected scores, renormalised."""
    from mini_sglang_amd import mixops

    torch.manual_seed(0)
    T, W, E, top, G, keep = 33, 40, 12, 3, 4, 2
    h = torch.randn(T, W)
    router = torch.randn(E, W) * 0.3
    bias = -2.0 - torch.rand(E)
    r = {"experts": E, "top": top, "groups": {"count": G, "keep": keep}}
    idx, wt = O.route(h.double(), r, {"p.router": router.double(), "p.correction": bias.double()}, "p.")
    ids, w = mixops.route(h.to(dev), router.to(dev), bias.to(dev), top, G, keep)
    order = idx.sort(1)
    mine = ids.cpu().long().sort(1)
    assert torch.equal(order.values, mine.values)
    assert torch.allclose(wt.gather(1, order.indices), w.cpu().double().gather(1, mine.indices), atol=1e-6)
    assert torch.allclose(w.sum(1).cpu(), torch.ones(T), atol=1e-5)


def test_grouped_product_and_bucketing(dev):
    """The segmented / gathered product behind the expert layers against a loop of torch products, ragged sizes."""
    from mini_sglang_amd import mixops

    torch.manual_seed(1)
    T, top, E, W, F = 37, 3, 5, 50, 70
    ids = torch.stack([torch.randperm(E)[:top] for _ in range(T)]).to(torch.int32)
    seg, perm = mixops.moe_sort(ids.to(dev), E)
    seg_h, perm_h = seg.cpu().tolist(), perm.cpu().tolist()
    flat = ids.flatten().tolist()
    assert seg_h[0] == 0 and seg_h[-1] == T * top
    for e in range(E):
        mine = perm_h[seg_h[e]: seg_h[e + 1]]
        assert mine == [i for i, x in enumerate(flat) if x == e]
    h, up = torch.randn(T, W), torch.randn(E, F, W)
    act = torch.zeros(T * top, F, device=dev)
    mixops.gemm_nt(act, h.to(dev), up.to(dev), T * top, F, W, lda=W, ldb=W, ldc=F, groups=E, b_gs=F * W, seg=seg, a_rows=perm,
                   a_div=top, act=mixops.ACT_RELU2)
    y = torch.zeros(T, top, W, device=dev)
    down = torch.randn(E, W, F)
    mixops.gemm_nt(y, act, down.to(dev), T * top, W, F, lda=F, ldb=F, ldc=W, groups=E, b_gs=W * F, seg=seg, c_rows=perm)
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            a = torch.relu(up[e].double() @ h[t].double()) ** 2
            assert torch.allclose(y[t, k].cpu().double(), down[e].double() @ a, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("M,N,K", [(70, 50, 37), (200, 256, 64), (1, 130, 96), (129, 127, 264)])
@pytest.mark.parametrize("a_dtype,c_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                             (torch.float32, torch.bfloat16)], ids=["bf16", "bf16-to-fp32", "fp32-a"])
def test_matrix_core_product(dev, M, N, K, a_dtype, c_dtype):
    """16-bit weights take the matrix-core kernel: sizes off every tile and vector boundary, per-head groups laid out side by
    side in one row (the latent-attention products), fp32 left operand rounded on the way in."""
    from mini_sglang_amd import mixops

    torch.manual_seed(M + N + K)
    G = 3
    a = torch.randn(M, G * K + 5).to(a_dtype)
    b = torch.randn(G, N, K).to(torch.bfloat16)
    c = torch.zeros(M, G * N + 3, dtype=c_dtype, device=dev)
    mixops.gemm_nt(c, a.to(dev), b.to(dev), M, N, K, lda=a.stride(0), ldb=K, ldc=c.stride(0), groups=G, a_gs=K, b_gs=N * K, c_gs=N)
    for g in range(G):
        ag = a[:, g * K: (g + 1) * K].to(torch.bfloat16).double()
        ref = ag @ b[g].double().T
        got = c[:, g * N: (g + 1) * N].cpu().double()
        tol = 2e-2 if c_dtype == torch.bfloat16 else 1e-4
        assert float((got - ref).abs().max() / ref.abs().max()) < tol, g
    assert float(c[:, G * N:].abs().max()) == 0.0


def test_expert_products_bf16(dev):
    """The expert path in 16 bits (matrix cores, gathered rows in, scattered rows out, ReLU^2 between), segments of very
    unequal length including empty ones."""
    from mini_sglang_amd import mixops

    torch.manual_seed(3)
    T, top, E, W, F = 300, 2, 7, 72, 136
    ids = torch.randint(0, 3, (T, top), dtype=torch.int32)
    ids[:5, 0] = 6  # expert 6: five rows; experts 3..5: none
    seg, perm = mixops.moe_sort(ids.to(dev), E)
    h = torch.randn(T, W).to(torch.bfloat16)
    up, down = (torch.randn(E, F, W) * W ** -0.5).to(torch.bfloat16), (torch.randn(E, W, F) * F ** -0.5).to(torch.bfloat16)
    act = torch.zeros(T * top, F, dtype=torch.bfloat16, device=dev)
    mixops.gemm_nt(act, h.to(dev), up.to(dev), T * top, F, W, lda=W, ldb=W, ldc=F, groups=E, b_gs=F * W, seg=seg, a_rows=perm,
                   a_div=top, act=mixops.ACT_RELU2)
    y = torch.zeros(T, top, W, dtype=torch.bfloat16, device=dev)
    mixops.gemm_nt(y, act, down.to(dev), T * top, W, F, lda=F, ldb=F, ldc=W, groups=E, b_gs=W * F, seg=seg, c_rows=perm)
    yh = y.cpu().double()
    for t in range(0, T, 7):
        for k in range(top):
            e = int(ids[t, k])
            a = (torch.relu(up[e].double() @ h[t].double()) ** 2).to(torch.bfloat16).double()
            ref = down[e].double() @ a
            assert float((yh[t, k] - ref).abs().max()) < 2e-2 * float(ref.abs().max()) + 1e-3, (t, k)


@pytest.mark.parametrize("n_keys", [1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 300])
@pytest.mark.parametrize("dtype,splits", [(torch.float32, 1), (torch.bfloat16, 1), (torch.bfloat16, 3)], ids=["fp32", "bf16", "bf16-split"])
def test_latent_attention_far_key_takes_all(dev, n_keys, dtype, splits):
    """One key far back (the first, or one on a page border) is made to win the softmax for one head while another head
    looks at the newest key: the output must be that key's latent.  Key counts sit on both sides of the kernels' key tiles
    and of the page size; the page table is shuffled; the 16-bit cache takes the matrix-core kernel, also with the keys
    cut into ranges that are merged afterwards (some of them empty)."""
    from mini_sglang_amd import mixops

    torch.manual_seed(n_keys)
    H, R, r, page = 3, 20, 6, 16
    slots = 512
    cache = torch.randn(slots, R + r).to(dtype)
    table = torch.randperm(slots)[: ((n_keys + page - 1) // page) * page].to(torch.int32).view(1, -1)
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32, device=dev)
    for far in sorted({0, min(n_keys - 1, 15), min(n_keys - 1, 16), n_keys // 2}):
        q = torch.randn(1, H, R + r) * 0.1
        cache[table[0, far]] *= 1.5
        q[0, 0] = 40.0 * cache[table[0, far]].float() / cache[table[0, far]].float().norm()
        q[0, 1] = 40.0 * cache[table[0, n_keys - 1]].float() / cache[table[0, n_keys - 1]].float().norm()
        out = torch.zeros(1, H, R, device=dev)
        mixops.latent_attn(out, q.to(dev), cache.to(dev), table.to(dev), i32(0), i32(n_keys), i32(0, 1), 1, R, 1.0, splits=splits)
        keys = cache[table[0, :n_keys].long()].double()
        qq = q[0].to(dtype).double()
        ref = torch.softmax(qq @ keys.T, -1) @ keys[:, :R]
        assert torch.allclose(out[0].cpu().double(), ref, atol=2e-5 if dtype == torch.float32 else 3e-2)


def test_latent_attention_matrix_core_batch(dev):
    """The matrix-core kernel on a mixed batch: a long portion with cached keys before it, single tokens, a short portion;
    more heads than one 16-row tile, key and value widths off the tile sizes."""
    from mini_sglang_amd import mixops

    torch.manual_seed(11)
    H, R, r = 20, 72, 24
    q_lens, k_lens = [70, 1, 5, 1], [200, 333, 5, 1]
    slots = 2048
    cache = (torch.randn(slots, R + r) * 0.5).to(torch.bfloat16)
    table = torch.randperm(slots)[: 4 * 352].to(torch.int32).view(4, 352)
    T = sum(q_lens)
    q = (torch.randn(T, H, R + r) * 0.3)
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
    out = torch.zeros(T, H, R, device=dev)
    mixops.latent_attn(out, q.to(dev), cache.to(dev), table.to(dev), i32([0, 1, 2, 3]), i32(k_lens), i32(cu), 4, R, 0.11)
    for b in range(4):
        keys = cache[table[b, : k_lens[b]].long()].double()
        for t in range(q_lens[b]):
            pos = k_lens[b] - q_lens[b] + t
            sc = q[cu[b] + t].to(torch.bfloat16).double() @ keys[: pos + 1].T * 0.11
            ref = torch.softmax(sc, -1) @ keys[: pos + 1, :R]
            got = out[cu[b] + t].cpu().double()
            assert float((got - ref).abs().max()) < 2e-2, (b, t)


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


@pytest.mark.parametrize("sizes", [[2], [3, 2, 5], [16], [15, 17], [64, 1, 63, 2], [33, 1, 1, 1, 7]])
def test_portions_fp32(sizes):
    eng_state = engine_for(FULL, torch.float32)
    toks = tokens_of(131, FULL["vocab"], 6)
    check(eng_state, FULL, alone("a", toks, sizes), {"a": toks}, FP32_TOL)


def test_long_portions_run_as_parallel_chunks_fp32():
    """Portions long enough for the recurrent layers to cut them into pieces (states joined by a scan): first a long portion
    from position 0, then a single token, then a long portion that continues from a carried state, beside a short request;
    lengths off the piece size."""
    eng_state = engine_for(FULL, torch.float32, max_tokens=1024)
    a, b = tokens_of(700, FULL["vocab"], 30), tokens_of(6, FULL["vocab"], 31)
    steps = [[("a", a[:300], False)], [("a", a[300:301], False), ("b", b[:5], False)], [("b", b[5:], True), ("a", a[301:], True)]]
    got = check(eng_state, FULL, steps, {"a": a, "b": b}, FP32_TOL)
    whole = replay(eng_state[0], alone("a", a, [257, 443]))["a"]
    assert rel(got["a"], whole) < 2e-5


def test_long_decoding_fp32():
    """A short prompt, then 260 tokens one by one: the recurrent state and the latent rows carry everything."""
    cfg = config([lit(mlp=moe()), lat(mlp=None), lit(heads=2, dim=12, vdim=20)])
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
    """A pool of 8 pages and two request rows: every request after the first runs on pages and on a state slot that still
    hold another request's rows and state; a request that ends frees them for the one admitted in the next step."""
    cfg = config([lit(decay=[0.999, 0.99, 0.9, 1.0]), lat(), lit(heads=2, dim=8, vdim=8, mlp=moe())])
    eng_state = engine_for(cfg, torch.float32, max_tokens=128, rows=2)
    seqs = {i: tokens_of(n, cfg["vocab"], 40 + k) for k, (i, n) in enumerate([("a", 60), ("b", 64), ("c", 50), ("d", 33), ("e", 64)])}
    steps = [[("a", seqs["a"][:40], False), ("b", seqs["b"][:30], False)],
             [("a", seqs["a"][40:], True), ("b", seqs["b"][30:], True)],
             [("c", seqs["c"][:20], False)],
             [("c", seqs["c"][20:], True), ("d", seqs["d"][:10], False)],
             [("d", seqs["d"][10:], True)],
             [("e", seqs["e"], True)]]
    check(eng_state, cfg, steps, seqs, FP32_TOL)


def test_other_orders_and_sizes_bf16():
    """Another order of layers, widths that are not powers of two, one expert per token, borrowed keys right after their
    owner: the 16-bit path end to end."""
    cfg = config([lat(heads=2, dim=12, rot_dim=4, vdim=20, kv_rank=36, mlp=moe(experts=3, top=1, ff=20, count=0)),
                  lat(kv_from=0, heads=4, dim=12, rot_dim=4, vdim=8, kv_rank=36), lit(heads=3, dim=12, vdim=28, mlp=moe())],
                 width=72, vocab=101, alpha=0.9, eps=1e-6)
    toks = tokens_of(120, cfg["vocab"], 10)
    check(engine_for(cfg, torch.bfloat16), cfg, alone("a", toks, [50, 1, 1, 30, 2, 36]), {"a": toks}, BF16_TOL, allow=0.1)


# ----------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("graphs", [None, [1, 2, 4]], ids=["eager", "graphs"])
def test_greedy_generation_through_the_scheduler(graphs):
    """OfflineRunner.generate (chunked prefill with a small budget, continuous decode, the sampler's argmax, captured
    decode graphs) against greedy decoding with the oracle; a step whose two best logits are closer than the fp32 tolerance
    ends the comparison for that request."""
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


def test_sampled_generation_runs():
    """Temperature / top-k / top-p draws through the same path: tokens in range and of the asked length."""
    from mini_sglang_amd.core import SamplingParams
    from mini_sglang_amd.offline import OfflineRunner

    eng, _ = engine_for(FULL, torch.bfloat16, max_tokens=512, graphs=[1, 2])
    run = OfflineRunner(eng, max_extend_tokens=64, seed=3)
    prompts = [tokens_of(n, FULL["vocab"], 80 + n) for n in (5, 20)]
    run.generate(prompts, [SamplingParams(temperature=0.8, top_k=10, top_p=0.9, max_tokens=6, ignore_eos=True)] * 2)
    for st in run.last_states:
        out = run.output_ids(st)
        assert len(out) == 6 and all(0 <= t < FULL["vocab"] for t in out)


def test_trace_command_line(tmp_path):
    """bin/trace_run end to end in its own process: a checkpoint folder written here (config.json + safetensors, widths that
    are no multiple of 16 so that some projections leave the library), recorded steps on stdin, logits files and `done` lines
    out; fp32 against the restatement, and float32 refused for nothing."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np
    from safetensors.torch import save_file

    from mini_sglang_amd.hybrid import HybridConfig, HybridDecoder

    cfg = config([lat(heads=3, dim=10, rot_dim=6, vdim=14, kv_rank=22, mlp=moe(experts=6, top=2, ff=26, count=3, keep=2)),
                  lit(heads=3, dim=10, vdim=18), lat(kv_from=0, heads=2, dim=10, rot_dim=6, vdim=30, kv_rank=22)], width=100, vocab=131)
    model = HybridDecoder(HybridConfig.from_json(cfg), dtype=torch.bfloat16, device=torch.device("cpu"), seed=9, max_position=64)
    state = model.export_state()
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
