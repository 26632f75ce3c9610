"""Host-side pieces of the hybrid decoder family: configuration reader, registry, rotary table, checkpoint round trip, and
the plain restatement's own consistency (its recurrence carried over a cut equals the whole; its router on a hand-made case)."""
from __future__ import annotations

import math

import pytest
import torch

import hybrid_oracle as O
from mini_sglang_amd.hybrid import HybridConfig, HybridDecoder, rotary_table
from mini_sglang_amd.kvcache import HybridCache
from mini_sglang_amd import registry


def _cfg():
    rot = {"base": 5000.0, "dims": 8, "scaling": {"factor": 4.0, "fast": 16.0, "original": 64, "slow": 2.0}}
    lat = {"heads": 3, "dim": 24, "rot_dim": 8, "vdim": 40, "kv_rank": 48, "rot": rot, "scale": 0.17}
    mlp = {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}
    return {"architecture": "Nidorax", "norm": {"eps": 1e-5}, "postln_alpha": 1.7, "vocab": 80, "width": 48, "layers": [
        {"type": "lightning", "mixer": {"heads": 2, "dim": 8, "vdim": 24, "decay": [0.9, 0.99]}, "mlp": mlp},
        {"type": "latent_attention", "mixer": lat, "mlp": None},
        {"type": "latent_attention", "mixer": dict(lat, kv_from=1, heads=5), "mlp": dict(mlp, router={"experts": 4, "top": 1})}]}


def test_config_reader_and_registry():
    raw = _cfg()
    cfg = HybridConfig.from_json(raw)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.num_layers, cfg.postln_alpha) == (80, 48, 3, 1.7)
    a, b, c = cfg.layers
    assert a.kind == "lightning" and a.decay == (0.9, 0.99) and (a.mlp.groups, a.mlp.keep) == (3, 2)
    assert b.kv_from is None and b.mlp is None and b.rot_dims == 8 and dict(b.rot_scaling)["factor"] == 4.0
    assert c.kv_from == 1 and c.heads == 5 and (c.mlp.groups, c.mlp.keep, c.mlp.top) == (1, 1, 1)
    assert registry.architecture_of(raw) == "Nidorax" and registry.model_class(cfg) is HybridDecoder
    assert registry.architecture_of({"architectures": ["Qwen3ForCausalLM"]}) == "Qwen3ForCausalLM"
    with pytest.raises(ValueError):
        registry.architecture_of({"architectures": ["Nope"]})
    bad = _cfg()
    bad["layers"][2]["mixer"]["kv_from"] = 0  # a lightning layer caches no keys
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)
    bad = _cfg()
    bad["layers"][0]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        HybridConfig.from_json(bad)


def test_dense_config_from_hf_names():
    cfg = registry.dense_config_from_hf({"model_type": "qwen3", "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128,
                                         "hidden_size": 1024, "vocab_size": 1000, "intermediate_size": 3072, "num_hidden_layers": 2,
                                         "rope_theta": 1e6, "tie_word_embeddings": True})
    assert cfg.qk_norm and cfg.num_kv_heads == 8 and cfg.rope_base == 1e6 and cfg.tie_word_embeddings


@pytest.mark.parametrize("scaled", [True, False])
def test_rotary_table_matches_the_restatement(scaled):
    raw = _cfg()
    if not scaled:
        del raw["layers"][1]["mixer"]["rot"]["scaling"]
    spec = HybridConfig.from_json(raw).layers[1]
    table = rotary_table(spec, 300, "cpu")
    f, amp = O.rot_frequencies(raw["layers"][1]["mixer"]["rot"])
    ang = torch.arange(300, dtype=torch.float64)[:, None] * f
    ref = torch.cat([ang.cos() * amp, ang.sin() * amp], -1)
    assert table.shape == (300, 8) and float((table.double() - ref).abs().max()) < 1e-7
    assert (amp == 1.0) == (not scaled)


def test_checkpoint_round_trip_and_cache_layout():
    cfg = HybridConfig.from_json(_cfg())
    a = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=1, max_position=64)
    b = HybridDecoder(cfg, dtype=torch.float32, device=torch.device("cpu"), seed=2, max_position=64)
    state = a.export_state()
    assert state["l1.mix.dkv"].shape == (48 + 8, 48) and state["l2.mix.uk"].shape == (5 * 24, 48) and "l2.mix.dkv" not in state
    assert state["l0.mlp.e5.up"].shape == (40, 48) and "l1.norm2" not in state
    b.load_state(state)
    for (k, u), v in zip(state.items(), b.export_state().values()):
        assert torch.equal(u, v), k
    cache = HybridCache(cfg.layers, num_pages=5, page_size=4, state_rows=3, dtype=torch.float32, device=torch.device("cpu"))
    assert cache.latent_rows(1).shape == (20, 56) and cache.latent_rows(2) is cache.latent_rows(1) and not cache.owns_latent(2)
    assert cache.state(0).shape == (3, 2, 8, 24) and cache.state(0).dtype == torch.float32
    assert HybridCache.bytes_per_page(cfg.layers, 4, torch.bfloat16) == 56 * 2 * 4


def test_restatement_recurrence_carries_over_a_cut():
    torch.manual_seed(0)
    m = {"heads": 2, "dim": 4, "vdim": 6, "decay": [0.7, 0.99]}
    w = {"p.q": torch.randn(8, 10).double(), "p.k": torch.randn(8, 10).double(), "p.v": torch.randn(12, 10).double(),
         "p.g": torch.randn(12, 10).double(), "p.o": torch.randn(10, 12).double(), "p.norm": torch.rand(12).double()}
    h = torch.randn(9, 10).double()
    whole, S = O.lightning(h, m, w, "p.", 1e-6)
    first, S1 = O.lightning(h[:4], m, w, "p.", 1e-6)
    rest, S2 = O.lightning(h[4:], m, w, "p.", 1e-6, state=S1)
    assert torch.allclose(torch.cat([first, rest]), whole, atol=1e-12) and torch.allclose(S, S2, atol=1e-12)


def test_restatement_router_by_hand():
    # softmax scores fixed through a one-hot input; groups of two; corrections make group 1 best although its raw scores are not
    r = {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}
    z = torch.tensor([[2.0, 1.0, 0.5, 0.0]], dtype=torch.float64)
    w = {"p.router": torch.eye(4, dtype=torch.float64), "p.correction": torch.tensor([0.0, 0.0, 0.9, -0.5], dtype=torch.float64)}
    idx, wt = O.route(z, r, w, "p.")
    s = torch.softmax(z, -1)[0]
    assert sorted(idx[0].tolist()) == [2, 3]
    assert math.isclose(float(wt.sum()), 1.0, rel_tol=1e-12)
    assert torch.allclose(wt[0].sort().values, (s[[2, 3]] / s[[2, 3]].sum()).sort().values)
