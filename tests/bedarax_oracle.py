"""Plain, slow restatement of the Bedarax design in torch on the CPU (test infrastructure only).

One function per mechanism, written from the equations and sharing no code with the product path: whole sequences, no
cache, no batching, a token-by-token loop wherever the design has a recurrence.  `dtype` float64 gives the yardstick the
kernels are compared with; nothing here rounds to 16 bits.

Notation: W = residual width, H = heads, G = key/value heads (query head h reads group h // (H / G)), d = query/key size
per head, dv = value size per head, E = experts.  Weights are a dict name -> tensor with the checkpoint's names.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# --------------------------------------------------------------------------------------- windowed attention with mixed heads
def mixed_head_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, v_first: Optional[torch.Tensor]):
    """h [T, W] -> (output [T, W], the values this layer caches [T, G, dv]).  Scores of all heads are mixed by the H x H
    table before the softmax; key j is visible from i when 0 <= i - j < window; each head's output is scaled by its own
    sigmoid gate.  `v_first` (the values of the first value-mixing layer) is blended in when given."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = (h @ w["v"].T).view(T, G, dv)
    if v_first is not None:
        lam = w["vmix"].reshape(())
        v = (1.0 - lam) * v + lam * v_first
    rep = H // G
    raw = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, dim=1)) * float(m["scale"])
    s = torch.einsum("hg,gij->hij", w["talk"], raw)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i)
    window = (m.get("mask") or {}).get("size")
    if window is not None:
        seen = seen & (i - j < int(window))
    s = s.masked_fill(~seen[None], -math.inf)
    p = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhe->ihe", p, v.repeat_interleave(rep, dim=1))
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w["o"].T, v


# --------------------------------------------------------------------------------------- delta-rule recurrences
def short_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1) + j, c]) with zeros before the sequence."""
    n = taps.shape[1]
    pad = torch.cat([torch.zeros(n - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(n):
        y = y + pad[j: j + x.shape[0]] * taps[:, j][None, :]
    return silu(y)


def unit_vectors(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """q, k [T, H, d], v [T, H, dv], beta [T, H], decay [T, H] or [T, H, d] -> o [T, H, dv].  Per head, per token:
    S <- decay * S (rows = key channels), u = beta (v - S^T k), S <- S + k u^T, o = S^T q."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype)
    out = []
    for t in range(T):
        g = decay[t]
        S = S * (g[:, None, None] if g.dim() == 1 else g[:, :, None])
        u = beta[t][:, None] * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out.append(torch.einsum("hde,hd->he", S, q[t]))
    return torch.stack(out)


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, per_channel: bool) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    rep = H // G
    q = short_conv_silu(h @ w["q"].T, w["q.conv"]).view(T, G, d)
    k = short_conv_silu(h @ w["k"].T, w["k.conv"]).view(T, G, d)
    v = short_conv_silu(h @ w["v"].T, w["v.conv"]).view(T, H, dv)
    q = (unit_vectors(q) * d ** -0.5).repeat_interleave(rep, dim=1)
    k = unit_vectors(k).repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(h @ w["b"].T)
    rate = torch.exp(w["A_log"])
    if per_channel:
        a = ((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, d)
        decay = torch.exp(-rate[None, :, None] * F.softplus(a))
        gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T)
    else:
        decay = torch.exp(-rate[None, :] * F.softplus(h @ w["a"].T + w["dt_bias"]))
        gate = silu(h @ w["g"].T)
    o = delta_rule(q, k, v, beta, decay)
    o = rms_unit(o, eps) * w["norm"][None, None, :] * gate.view(T, H, dv)
    return o.reshape(T, H * dv) @ w["o"].T


# --------------------------------------------------------------------------------------- feed-forwards
def poly_norm_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    z = h @ w["up"].T
    a, b, c, e = w["act"].unbind(0)
    act = a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e
    return act @ w["down"].T


def route_top_logits(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor, top: int):
    """-> (expert ids [T, top] by descending logit, softmax over the chosen logits [T, top])."""
    z = h @ router.T + bias
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def gated_experts_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    idx, wt = route_top_logits(h, w["router"], w["router.b"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(idx[t, c])
            y = (silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T
            out[t] = out[t] + wt[t, c] * y
    assert E == sum(1 for k in w if k.endswith(".up"))
    return out


# --------------------------------------------------------------------------------------- the stack
def sub(weights: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens, dtype=torch.float64, layer_outputs: Optional[List] = None):
    """tokens: ids of ONE sequence -> logits [T, vocab]; layer_outputs (if a list) receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    W = {k: v.to(dtype) for k, v in weights.items()}
    x = norm(W["embed"][torch.as_tensor(tokens, dtype=torch.long)], W["embed.norm"], eps)
    history = [x]
    v_first = None
    for i, entry in enumerate(cfg["layers"]):
        m, mlp, kind = entry["mixer"], entry.get("mlp"), entry["type"]
        h = norm(x, W[f"l{i}.norm1"], eps)
        mw = sub(W, f"l{i}.mix.", dtype)
        if kind == "attention":
            y, v = mixed_head_attention(h, mw, m, v_first if m.get("v_mix") else None)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif kind in ("delta", "channel_delta"):
            y = delta_mixer(h, mw, m, eps, per_channel=kind == "channel_delta")
        else:
            raise ValueError(kind)
        x = x + y
        if mlp is not None:
            h = norm(x, W[f"l{i}.norm2"], eps)
            fw = sub(W, f"l{i}.mlp.", dtype)
            x = x + (poly_norm_ff(h, fw, eps) if mlp["kind"] == "dense" else gated_experts_ff(h, fw, mlp))
        history.append(x)
        c = W[f"l{i}.dwa"]
        x = sum(c[j] * history[j] for j in range(i + 2))
        if layer_outputs is not None:
            layer_outputs.append(x)
    return norm(x, W["final.norm"], eps) @ W["head"].T
