"""Host-side pieces of the pre-norm hybrid decoder (Bedarax): configuration reader and registry, checkpoint round trip,
cache layout, the C ABI table against the header, and the restatement's own consistency.  No GPU."""
from __future__ import annotations

import ctypes as C
import json
import re
from pathlib import Path

import pytest
import torch

import bedarax_oracle as O

ROOT = Path(__file__).resolve().parent.parent


def _cfg():
    moe = {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 5, "top": 2}}
    return {"architecture": "Bedarax", "norm": {"eps": 1e-5}, "vocab": 50, "width": 24, "layers": [
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 0.4, "mask": {"size": 9}, "v_mix": True},
         "mlp": {"kind": "dense", "ff": 20}},
        {"type": "channel_delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 8, "conv": 3}, "mlp": moe},
        {"type": "delta", "mixer": {"heads": 2, "kv_heads": 2, "dim": 4, "vdim": 6, "conv": 2}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 6, "vdim": 10, "scale": 1.0, "v_mix": True}, "mlp": moe}]}


def test_config_reader_and_registry(tmp_path):
    from mini_sglang_amd.hybrid import DenseFfSpec, HybridConfig, HybridDecoder, MoeSpec, bedarax_config
    from mini_sglang_amd.registry import architecture_of, load_model_dir, model_class

    raw = _cfg()
    assert architecture_of(raw) == "Bedarax"
    cfg = bedarax_config(raw, {"l1.mix.a1": (5, 24), "l1.mix.g1": (7, 24)})
    assert isinstance(cfg, HybridConfig) and cfg.residual == "pre_norm_depth" and model_class(cfg) is HybridDecoder
    a, c, d, a2 = cfg.layers
    assert (a.kind, a.heads, a.kv_heads, a.window, a.v_mix, a.scale) == ("attention", 4, 2, 9, True, 0.4) and isinstance(a.mlp, DenseFfSpec)
    assert (c.kind, c.conv, c.decay_rank, c.gate_rank) == ("channel_delta", 3, 5, 7) and isinstance(c.mlp, MoeSpec)
    assert c.mlp.gated and c.mlp.pick == "logits" and (c.mlp.experts, c.mlp.top, c.mlp.ff) == (5, 2, 12)
    assert d.mlp is None and d.recurrent and a2.window == 0
    no_taps = _cfg()
    del no_taps["layers"][2]["mixer"]["conv"]  # a size config.json leaves out comes from the tensor's shape
    assert bedarax_config(no_taps, {"l2.mix.q.conv": (8, 5)}).layers[2].conv == 5 and bedarax_config(no_taps).layers[2].conv == 1
    bad = _cfg()
    bad["layers"][3]["mixer"]["vdim"] = 12  # value-mixing layers must agree
    with pytest.raises(ValueError):
        bedarax_config(bad)
    bad = _cfg()
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    with pytest.raises(ValueError):
        bedarax_config(bad)
    # a folder: the inner sizes come from the checkpoint's header
    from safetensors.torch import save_file

    model = HybridDecoder(cfg, dtype=torch.bfloat16, device=torch.device("cpu"), seed=1)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    save_file(model.export_state(), str(tmp_path / "model.safetensors"))
    cfg2, name = load_model_dir(tmp_path)
    assert name == "Bedarax" and cfg2 == cfg


def test_checkpoint_round_trip_and_cache_layout():
    from mini_sglang_amd.hybrid import HybridDecoder, bedarax_config
    from mini_sglang_amd.kvcache import HybridCache

    cfg = bedarax_config(_cfg())
    a = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=1)
    b = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=2)
    state = a.export_state()
    assert state["l0.dwa"].shape == (2,) and state["l3.dwa"].shape == (5,) and state["l0.mix.vmix"].shape == ()
    assert state["l1.mix.q.conv"].shape == (6, 3) and state["l1.mix.v.conv"].shape == (16, 3) and state["l1.mix.dt_bias"].shape == (12,)
    assert state["l2.mix.a"].shape == (2, 24) and state["l2.mix.dt_bias"].shape == (2,) and state["l0.mlp.act"].shape == (4,)
    assert state["l1.mlp.e4.gate"].shape == (12, 24) and state["l1.mlp.router.b"].shape == (5,) and state["head"].shape == (50, 24)
    b.load_state(state)
    for k, v in b.export_state().items():
        assert torch.allclose(v.float(), state[k].float(), rtol=1e-6, atol=1e-7), k
    cache = HybridCache(cfg.layers, num_pages=4, page_size=8, state_rows=3, dtype=torch.bfloat16, device=torch.device("cpu"))
    k, v = cache.kv_rows(0)
    assert k.shape == (32, 12) and v.shape == (32, 20) and k.dtype == torch.bfloat16
    assert cache.state(1).shape == (3, 2, 6, 8) and cache.state(1).dtype == torch.float32
    assert cache.conv_state(1).shape == (3, 2, 2 * 6 + 16) and cache.conv_state(2).shape == (3, 1, 2 * 2 * 4 + 12)
    assert HybridCache.bytes_per_page(cfg.layers, 8, torch.bfloat16) == 2 * 8 * (2 * 16 + 2 * 16)


def test_abi_table_matches_the_header():
    from mini_sglang_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / "msgl_mix.h").read_text(), flags=re.S)
    seen = 0
    for m in re.finditer(r"(?:int|const char\*) (msgl_mix_\w+)\(([^)]*)\)", text):
        params = [p.strip() for p in m.group(2).split(",") if p.strip() != "void"]
        kinds = [C.c_void_p if "*" in p else C.c_int64 if p.startswith("int64_t") else C.c_float if p.startswith("float") else C.c_int
                 for p in params]
        assert _lib.MIX_SIGNATURES[m.group(1)][1] == kinds, m.group(1)
        seen += 1
    assert seen == len(_lib.MIX_SIGNATURES)


def test_restatement_carries_over_a_cut():
    """The recurrence and the convolution of the restatement, fed in two pieces with their state handed over by hand, give
    what the whole sequence gives."""
    g = torch.Generator().manual_seed(3)
    T, H, d, dv = 17, 2, 5, 7
    q, k = (torch.randn(T, H, d, generator=g, dtype=torch.float64) for _ in range(2))
    v = torch.randn(T, H, dv, generator=g, dtype=torch.float64)
    beta, decay = torch.rand(T, H, generator=g, dtype=torch.float64), torch.rand(T, H, d, generator=g, dtype=torch.float64)
    whole = O.delta_rule(q, k, v, beta, decay)
    S = torch.zeros(H, d, dv, dtype=torch.float64)
    rows = []
    for t in range(T):  # the same rule written out per head
        for h in range(H):
            S[h] = decay[t, h][:, None] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ k[t, h])
            S[h] = S[h] + torch.outer(k[t, h], u)
        rows.append(torch.stack([S[h].T @ q[t, h] for h in range(H)]))
    assert torch.allclose(torch.stack(rows), whole, atol=1e-12)
    x, taps = torch.randn(T, 6, generator=g, dtype=torch.float64), torch.randn(6, 4, generator=g, dtype=torch.float64)
    full = O.short_conv_silu(x, taps)
    tail = O.short_conv_silu(torch.cat([x[7:10], x[10:]]), taps)[3:]  # three inputs of history = taps - 1
    assert torch.allclose(full[10:], tail, atol=1e-12)


def test_restatement_router_and_activation_by_hand():
    h = torch.tensor([[1.0, 0.0], [0.0, 2.0]], dtype=torch.float64)
    router = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=torch.float64)
    bias = torch.tensor([0.0, 0.5, -0.25], dtype=torch.float64)
    idx, wt = O.route_top_logits(h, router, bias, 2)
    assert idx.tolist() == [[0, 2], [1, 2]]
    assert torch.allclose(wt[0], torch.softmax(torch.tensor([1.0, 0.75], dtype=torch.float64), 0))
    z = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    w = {"up": torch.eye(2, dtype=torch.float64), "down": torch.eye(2, dtype=torch.float64),
         "act": torch.tensor([2.0, 0.5, 0.25, 0.1], dtype=torch.float64)}
    r1, r2, r3 = (12.5) ** 0.5, ((81 + 256) / 2) ** 0.5, ((729 + 4096) / 2) ** 0.5
    want = torch.tensor([[2 * 3 / r1 + 0.5 * 9 / r2 + 0.25 * 27 / r3 + 0.1, 2 * -4 / r1 + 0.5 * 16 / r2 + 0.25 * -64 / r3 + 0.1]])
    assert torch.allclose(O.poly_norm_ff(z, w, 0.0), want.double(), atol=1e-12)
