"""Hybrid decoder stack: latent-attention layers and linear-recurrence ("lightning") layers with routed-expert
feed-forwards and norm-after-sum residuals (the Nidorax design; any order and any sizes, all read from its config.json).

Per layer   x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ff(x)),  norm(s) = s / sqrt(mean(s^2) + eps) * (1 + w).
The residual stream x lives in fp32; `h` is its copy in the model dtype that the projections read.

latent attention   q = W_q h per head [d unrotated | r rotated];  W_dkv h = [latent (RMS-normed, weight dkv.norm) | one
                   rotated key part shared by the heads];  cached per token: the latent c and the rotated part (R + r numbers).
                   The per-head key W_uk c is never built: the query is carried into latent space once per token
                   (q_abs = W_uk^T q_unrotated, a grouped product over heads), scores are q_abs . c + q_r . k_r, the softmax-
                   weighted LATENT is accumulated and W_uv is applied to it afterwards (grouped product), so prefill portions
                   and decoded tokens read the same R + r numbers per key whatever the head count.  A layer with `kv_from`
                   reads the rows another layer wrote in the same forward.
lightning          S <- decay_h S + k v^T, o = S^T q with q, k, v = SiLU(projections); fp32 state per (request, head) in the
                   cache's state rows; heads concatenated, RMS-normed (plain weight), gated by sigmoid(W_g h).
feed-forward       fp32 router (softmax, bias-corrected choice, group-limited top-k) inside the launch of the norm before it
                   (short batches) or on product-kernel logits (long ones), (token, choice) pairs bucketed by expert on the
                   device, two segmented grouped products (up with ReLU^2, down), the weighted sum of a token's choices folded
                   into the norm that follows.

Kernels: csrc/seqmix.hip through mixops.py; plain projections through the library GEMM (mixops.linear).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch

from . import flashinfer_compat as fi
from . import mixops


@dataclass(frozen=True)
class MoeSpec:
    experts: int
    top: int
    ff: int
    groups: int = 1
    keep: int = 1


@dataclass(frozen=True)
class LayerSpec:
    kind: str                       # "latent_attention" | "lightning"
    heads: int
    dim: int                        # unrotated query/key size per head (lightning: query/key size)
    vdim: int
    rot_dim: int = 0
    kv_rank: int = 0
    kv_from: Optional[int] = None
    scale: float = 1.0
    rot_dims: int = 0               # how many entries of the rotated part turn
    rot_base: float = 10000.0
    rot_scaling: Optional[Tuple[Tuple[str, float], ...]] = None
    decay: Tuple[float, ...] = ()
    mlp: Optional[MoeSpec] = None


@dataclass(frozen=True)
class HybridConfig:
    """What a Nidorax config.json states, nothing else; `max_position` is the engine's sequence limit (the design has none)."""
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    rms_norm_eps: float
    postln_alpha: float
    max_position: int = 1 << 20
    name: str = "Nidorax"

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_json(cfg: Dict[str, Any], name: str = "Nidorax") -> "HybridConfig":
        layers: List[LayerSpec] = []
        for i, entry in enumerate(cfg["layers"]):
            m, mlp = entry["mixer"], entry.get("mlp")
            moe = None
            if mlp is not None:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                r, g = mlp["router"], mlp["router"].get("groups") or {}
                moe = MoeSpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(mlp["expert"]["ff"]),
                              groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))))
            if entry["type"] == "latent_attention":
                rot = m["rot"]
                sc = rot.get("scaling")
                layers.append(LayerSpec(
                    kind="latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]),
                    kv_from=None if m.get("kv_from") is None else int(m["kv_from"]), scale=float(m["scale"]),
                    rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot["base"]),
                    rot_scaling=None if not sc else tuple(sorted((k, float(v)) for k, v in sc.items())), mlp=moe))
            elif entry["type"] == "lightning":
                layers.append(LayerSpec(kind="lightning", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                        decay=tuple(float(x) for x in m["decay"]), mlp=moe))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {entry['type']!r}")
        for i, s in enumerate(layers):
            if s.kind == "latent_attention" and s.kv_from is not None:
                o = layers[s.kv_from] if 0 <= s.kv_from < i else None
                if o is None or o.kind != "latent_attention" or o.kv_from is not None or \
                        (o.kv_rank, o.rot_dim) != (s.kv_rank, s.rot_dim):
                    raise ValueError(f"layer {i}: kv_from = {s.kv_from} is not an earlier latent layer with its own keys of equal size")
            if s.kind == "lightning" and len(s.decay) != s.heads:
                raise ValueError(f"layer {i}: {len(s.decay)} decays for {s.heads} heads")
        return HybridConfig(vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=tuple(layers),
                            rms_norm_eps=float(cfg["norm"]["eps"]), postln_alpha=float(cfg["postln_alpha"]), name=name)


def rotary_table(spec: LayerSpec, max_position: int, device) -> torch.Tensor:
    """fp32 [max_position, rot_dims] = cos | sin of the layer's (scaled) rotary angles, amplitude folded in."""
    sc = dict(spec.rot_scaling) if spec.rot_scaling else None
    factor = sc["factor"] if sc else 1.0
    scaling = dict(rope_type="yarn", factor=factor, original_max_position_embeddings=sc["original"] if sc else 1.0,
                   beta_fast=sc["fast"] if sc else 2.0, beta_slow=sc["slow"] if sc else 1.0, hi_cap=spec.rot_dims - 1,
                   min_span=0.001, amplitude=0.1 * math.log(factor) + 1.0, float64_table=True)
    return fi.build_cos_sin_cache(spec.rot_dims, max_position, spec.rot_base, scaling, device=device)


class _Layer:
    __slots__ = ("spec", "w_in", "o", "norm1", "norm2", "uk_t", "uv", "c_norm", "cos_sin", "out_norm", "decay", "router",
                 "bias", "up", "down")

    def __init__(self, spec: LayerSpec) -> None:
        self.spec = spec
        for k in self.__slots__[1:]:
            setattr(self, k, None)


class HybridDecoder:
    ROUTE_FUSE_MAX_TOKENS = 128

    def __init__(self, cfg: HybridConfig, *, dtype: torch.dtype, device: torch.device, tp_rank: int = 0, tp_size: int = 1,
                 seed: int = 42, init_std: float = 0.02, max_position: Optional[int] = None, **_unused: Any) -> None:
        if tp_size != 1:
            raise NotImplementedError("the hybrid decoder runs on one rank (no tensor-parallel sharding of its layers yet)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"hybrid decoder: dtype {dtype} (bfloat16 or float32)")
        self.cfg, self.dtype, self.device = cfg, dtype, device
        self.tp_rank, self.tp_size = tp_rank, tp_size
        self.max_position = int(max_position or cfg.max_position)
        g = torch.Generator(device=device)
        g.manual_seed(seed)

        def w(*shape, std=init_std):  # seeded weights until a checkpoint is loaded
            return (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * std).to(dtype)

        W = cfg.hidden_size
        self.embed = w(cfg.vocab_size, W, std=1.0)
        self.final_norm = w(W, std=0.1)
        self.layers: List[_Layer] = []
        tables: Dict[tuple, torch.Tensor] = {}
        for spec in cfg.layers:
            L = _Layer(spec)
            H, d, dv = spec.heads, spec.dim, spec.vdim
            L.norm1 = w(W, std=0.1)
            if spec.kind == "latent_attention":
                r, R = spec.rot_dim, spec.kv_rank
                L.w_in = w(H * (d + r) + (0 if spec.kv_from is not None else R + r), W, std=W ** -0.5)
                L.uk_t = w(H, R, d, std=R ** -0.5)   # W_uk per head, transposed: q_abs = q_unrotated @ uk_t[h]^T
                L.uv = w(H, dv, R, std=R ** -0.5)
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.c_norm = None if spec.kv_from is not None else (1.0 + w(R, std=0.1).float()).to(dtype)
                key = (spec.rot_dims, spec.rot_base, spec.rot_scaling)
                if key not in tables:
                    tables[key] = rotary_table(spec, self.max_position, device)
                L.cos_sin = tables[key]
            else:
                L.w_in = w(2 * H * d + 2 * H * dv, W, std=W ** -0.5)  # q | k | v | gate
                L.o = w(W, H * dv, std=(H * dv) ** -0.5)
                L.out_norm = (1.0 + w(H * dv, std=0.1).float()).to(dtype)
                L.decay = torch.tensor(spec.decay, dtype=torch.float32, device=device)
            if spec.mlp is not None:
                m = spec.mlp
                L.norm2 = w(W, std=0.1)
                L.router = w(m.experts, W, std=W ** -0.5)
                L.bias = w(m.experts, std=0.01)
                L.up = w(m.experts, m.ff, W, std=W ** -0.5)
                L.down = w(m.experts, W, m.ff, std=m.ff ** -0.5)
            self.layers.append(L)

    # ------------------------------------------------------------------ weights
    def _tensors(self):
        yield self.embed
        yield self.final_norm
        for L in self.layers:
            for k in ("w_in", "o", "norm1", "norm2", "uk_t", "uv", "c_norm", "out_norm", "router", "bias", "up", "down"):
                t = getattr(L, k)
                if t is not None:
                    yield t

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._tensors())

    def streamed_bytes_per_step(self) -> int:
        return self.weight_bytes()

    def load_state(self, state: Dict[str, torch.Tensor]) -> None:
        """Overwrite the seeded weights with a checkpoint's tensors (names as in its TENSORS listing: 'embed', 'final.norm',
        'l<i>.norm1', 'l<i>.mix.<name>', 'l<i>.mlp.e<j>.up' ...), merging what one launch reads together: q | dkv, q | k | v | g,
        the experts of a layer stacked, W_uk split per head and transposed."""
        cfg = self.cfg

        def put(dst: torch.Tensor, src: torch.Tensor) -> None:
            if tuple(dst.shape) != tuple(src.shape):
                raise ValueError(f"checkpoint tensor of shape {tuple(src.shape)} where the config implies {tuple(dst.shape)}")
            dst.copy_(src.to(device=self.device, dtype=torch.float32).to(self.dtype))

        put(self.embed, state["embed"])
        put(self.final_norm, state["final.norm"])
        for i, L in enumerate(self.layers):
            s, p = L.spec, f"l{i}.mix."
            H, d, dv = s.heads, s.dim, s.vdim
            put(L.norm1, state[f"l{i}.norm1"])
            if s.kind == "latent_attention":
                parts = [state[p + "q"]] + ([] if s.kv_from is not None else [state[p + "dkv"]])
                put(L.w_in, torch.cat(parts, dim=0))
                put(L.uk_t, state[p + "uk"].view(H, d, s.kv_rank).transpose(1, 2).contiguous())
                put(L.uv, state[p + "uv"].view(H, dv, s.kv_rank))
                if s.kv_from is None:
                    put(L.c_norm, state[p + "dkv.norm"])
            else:
                put(L.w_in, torch.cat([state[p + "q"], state[p + "k"], state[p + "v"], state[p + "g"]], dim=0))
                put(L.out_norm, state[p + "norm"])
            put(L.o, state[p + "o"])
            if s.mlp is None and f"l{i}.norm2" in state:  # a layer without feed-forward that still norms a second time
                L.norm2 = torch.empty_like(L.norm1)
                put(L.norm2, state[f"l{i}.norm2"])
            if s.mlp is not None:
                q = f"l{i}.mlp."
                put(L.norm2, state[f"l{i}.norm2"])
                put(L.router, state[q + "router"])
                if (q + "correction") in state:
                    put(L.bias, state[q + "correction"])
                else:
                    L.bias = None
                put(L.up, torch.stack([state[f"{q}e{e}.up"] for e in range(s.mlp.experts)]))
                put(L.down, torch.stack([state[f"{q}e{e}.down"] for e in range(s.mlp.experts)]))

    def export_state(self) -> Dict[str, torch.Tensor]:
        """The inverse of load_state (checkpoint names, host tensors): what tests and tools hand to an independent implementation."""
        out = {"embed": self.embed, "final.norm": self.final_norm}
        for i, L in enumerate(self.layers):
            s, p = L.spec, f"l{i}.mix."
            H, d, dv = s.heads, s.dim, s.vdim
            out[f"l{i}.norm1"] = L.norm1
            if s.kind == "latent_attention":
                nq = H * (d + s.rot_dim)
                out[p + "q"] = L.w_in[:nq]
                if s.kv_from is None:
                    out[p + "dkv"], out[p + "dkv.norm"] = L.w_in[nq:], L.c_norm
                out[p + "uk"] = L.uk_t.transpose(1, 2).reshape(H * d, s.kv_rank)
                out[p + "uv"] = L.uv.reshape(H * dv, s.kv_rank)
            else:
                a, b = H * d, H * dv
                out[p + "q"], out[p + "k"], out[p + "v"], out[p + "g"] = L.w_in[:a], L.w_in[a:2 * a], L.w_in[2 * a:2 * a + b], L.w_in[2 * a + b:]
                out[p + "norm"] = L.out_norm
            out[p + "o"] = L.o
            if s.mlp is None and L.norm2 is not None:
                out[f"l{i}.norm2"] = L.norm2
            if s.mlp is not None:
                q = f"l{i}.mlp."
                out[f"l{i}.norm2"], out[q + "router"] = L.norm2, L.router
                if L.bias is not None:
                    out[q + "correction"] = L.bias
                for e in range(s.mlp.experts):
                    out[f"{q}e{e}.up"], out[f"{q}e{e}.down"] = L.up[e], L.down[e]
        return {k: v.detach().to("cpu").contiguous() for k, v in out.items()}

    def tune_gemms(self, batch_sizes, mode: str = "heuristic", log=None, prefill_tokens=()) -> List[dict]:
        return []  # the library's heuristic pick; the grouped products have one kernel

    # ------------------------------------------------------------------ forward
    def _latent(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        s, md, kv = L.spec, batch.attn_metadata, ctx.kv_cache
        T, H, d, r, R, dv = h.shape[0], s.heads, s.dim, s.rot_dim, s.kv_rank, s.vdim
        proj = mixops.linear(h, L.w_in)
        q_abs = torch.empty((T, H, R + r), dtype=torch.float32, device=h.device)
        rows = kv.latent_rows(i)
        own = s.kv_from is None
        mixops.latent_prep(proj, q_abs, rows if own else None, batch.out_loc if own else None, batch.positions, L.cos_sin,
                           L.c_norm, self.cfg.rms_norm_eps, H, d, r, R)
        mixops.gemm_nt(q_abs, proj, L.uk_t, T, R, d, lda=proj.stride(0), ldb=d, ldc=H * (R + r), groups=H, a_gs=d + r,
                       b_gs=R * d, c_gs=R + r)
        o_lat = torch.empty((T, H, R), dtype=torch.float32, device=h.device)
        # few query rows per request (decode, short portions): cut the keys into ranges so that the launch fills the chip
        splits = mixops.latent_attn_splits(md.batch, T, H, md.max_seqlen_k) if md.max_seqlen_q <= 16 else 1
        mixops.latent_attn(o_lat, q_abs, rows, ctx.page_table, md.req_rows, md.seq_lens, md.cu_seqlens_q, md.batch, R, s.scale,
                           splits=splits)
        o = torch.empty((T, H * dv), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(o, o_lat, L.uv, T, dv, R, lda=H * R, ldb=R, ldc=H * dv, groups=H, a_gs=R, b_gs=dv * R, c_gs=dv)
        return mixops.linear(o, L.o)

    def _lightning(self, i: int, L: _Layer, h: torch.Tensor, ctx: Any, batch: Any) -> torch.Tensor:
        s, md = L.spec, batch.attn_metadata
        T, H, d, dv = h.shape[0], s.heads, s.dim, s.vdim
        proj = mixops.linear(h, L.w_in)
        o = torch.empty((T, H * dv), dtype=torch.float32, device=h.device)
        mixops.lightning(o, proj, ctx.kv_cache.state(i), L.decay, md.cu_seqlens_q, md.seq_lens, md.req_rows, md.batch,
                         chunks=getattr(md, "chunks", None))
        gated = mixops.gated_norm(o, proj[:, 2 * H * d + H * dv:], L.out_norm, self.cfg.rms_norm_eps)
        return mixops.linear(gated, L.o)

    def _experts(self, L: _Layer, h: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """-> per-choice outputs [T, top, W] of the experts `ids` chose; the weighted sum over choices is the caller's norm's."""
        m, (T, W) = L.spec.mlp, h.shape
        seg, perm = mixops.moe_sort(ids, m.experts)
        n = T * m.top
        act = torch.empty((n, m.ff), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(act, h, L.up, n, m.ff, W, lda=W, ldb=W, ldc=m.ff, groups=m.experts, b_gs=m.ff * W, seg=seg, a_rows=perm,
                       a_div=m.top, act=mixops.ACT_RELU2)
        y = torch.empty((T, m.top, W), dtype=self.dtype, device=h.device)
        mixops.gemm_nt(y, act, L.down, n, W, m.ff, lda=m.ff, ldb=m.ff, ldc=W, groups=m.experts, b_gs=W * m.ff, seg=seg, c_rows=perm)
        return y

    def forward(self, ctx: Any, batch: Any, logits_out: Optional[torch.Tensor] = None, layer_outputs: Optional[list] = None) -> torch.Tensor:
        """-> logits [rows, vocab] in the model dtype: at `batch.logit_rows` (token indices) when set, else at every request's
        last token (prefill) or at every token (decode)."""
        cfg = self.cfg
        eps, alpha = cfg.rms_norm_eps, cfg.postln_alpha
        x, h = mixops.embed(self.embed, batch.input_ids)
        for i, L in enumerate(self.layers):
            y = self._latent(i, L, h, ctx, batch) if L.spec.kind == "latent_attention" else self._lightning(i, L, h, ctx, batch)
            m = L.spec.mlp
            # Few tokens (decode, short portions): the norm that closes the mixer's sum also routes its output -- router logits,
            # choice and weights leave the same launch.  Many tokens: every token re-reading the router weights costs more than
            # the launches it saves, so the logits come from the product kernel (weights reused across a 128-token tile).
            fuse = m is not None and h.shape[0] <= self.ROUTE_FUSE_MAX_TOKENS
            picks = mixops.postnorm(x, L.norm1, eps, y=y, alpha=alpha, x_out=x, h_out=h,
                                    route=(L.router, L.bias, m.top, m.groups, m.keep) if fuse else None)
            if m is not None and not fuse:
                picks = mixops.route(h, L.router, L.bias, m.top, m.groups, m.keep)
            if m is not None:
                y = self._experts(L, h, picks[0])
                mixops.postnorm(x, L.norm2, eps, y=y, gate=picks[1], alpha=alpha, x_out=x, h_out=h)
            elif L.norm2 is not None:
                mixops.postnorm(x, L.norm2, eps, alpha=alpha, x_out=x, h_out=h)
            if layer_outputs is not None:
                layer_outputs.append(x.clone())
        rows = getattr(batch, "logit_rows", None)
        if rows is None and batch.is_prefill:
            rows = batch.attn_metadata.get_last_indices(batch.size)
        if rows is not None:
            x = x.index_select(0, rows.to(torch.int64))
        hf = torch.empty(x.shape, dtype=self.dtype, device=x.device)
        mixops.postnorm(x, self.final_norm, eps, h_out=hf)
        if logits_out is not None and logits_out.shape == (hf.shape[0], cfg.vocab_size) and logits_out.dtype == self.dtype:
            return mixops.linear(hf, self.embed, out=logits_out)
        return mixops.linear(hf, self.embed)
