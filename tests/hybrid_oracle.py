"""Plain, slow restatement of the Nidorax design in torch on the CPU (test infrastructure only).

One function per mechanism, written from the equations and sharing no code with the product path: whole
sequences, no cache, no batching, every token of a sequence recomputed from the start.  `dtype` float64 gives
the yardstick the kernels are compared with; nothing here rounds to 16 bits.

Notation: W = residual width, H = heads, d = unrotated query/key size per head, r = rotated size, dv = value size,
R = latent size, E = experts.  Weights are a dict name -> tensor with the checkpoint's names.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_centered(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight is an offset from one."""
    return rms_unit(x, eps) * (1.0 + w)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# --------------------------------------------------------------------------------------- rotation
def rot_frequencies(rot: dict) -> Tuple[torch.Tensor, float]:
    """(angular frequency per pair [dims/2] float64, amplitude applied to cos and sin)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t: float) -> float:
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half_layout(x: torch.Tensor, pos: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [..., T, n >= dims]: the first `dims` entries rotated (entry i paired with i + dims/2), the rest kept."""
    dims = int(rot["dims"])
    f, amp = rot_frequencies(rot)
    ang = pos.to(torch.float64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * amp).to(x.dtype), (torch.sin(ang) * amp).to(x.dtype)
    u, v = x[..., : dims // 2], x[..., dims // 2: dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# --------------------------------------------------------------------------------------- mixers
def latent_kv(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, pos: torch.Tensor):
    """What a latent-attention layer caches: (latent c [T, R], rotated shared key part [T, r])."""
    R = int(m["kv_rank"])
    dkv = h @ w[p + "dkv"].T
    c = rms_unit(dkv[:, :R], eps) * w[p + "dkv.norm"]
    return c, rotate_half_layout(dkv[:, R:], pos, m["rot"])


def latent_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, pos: torch.Tensor,
                     c: torch.Tensor, kr: torch.Tensor) -> torch.Tensor:
    """h [T, W] -> [T, W]; c, kr are the (own or borrowed) cached latent and rotated key part."""
    T = h.shape[0]
    H, d, r, dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    qn, qr = q[..., :d], rotate_half_layout(q[..., d:].transpose(0, 1), pos, m["rot"]).transpose(0, 1)
    kn = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", qn, kn) + torch.einsum("ihr,jr->hij", qr, kr)) * float(m["scale"])
    keep = torch.tril(torch.ones(T, T, dtype=torch.bool))
    a = torch.softmax(s.masked_fill(~keep, float("-inf")), dim=-1)
    o = torch.einsum("hij,jhv->ihv", a, v).reshape(T, H * dv)
    return o @ w[p + "o"].T


def lightning(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float,
              state: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Token-by-token linear recurrence per head; returns (output [T, W], final state [H, d, dv])."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    silu = torch.nn.functional.silu
    q = silu(h @ w[p + "q"].T).view(T, H, d)
    k = silu(h @ w[p + "k"].T).view(T, H, d)
    v = silu(h @ w[p + "v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)
    S = torch.zeros(H, d, dv, dtype=h.dtype) if state is None else state.clone()
    out = torch.empty(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = rms_unit(out.reshape(T, H * dv), eps) * w[p + "norm"]
    y = y * torch.sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T, S


# --------------------------------------------------------------------------------------- feed-forward
def route(h: torch.Tensor, r: dict, w: Dict[str, torch.Tensor], p: str) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> (chosen experts [T, top] int64, their weights [T, top])."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    choice = s + w[p + "correction"] if (p + "correction") in w else s.clone()
    g = r.get("groups")
    if g:
        G, keep = int(g["count"]), int(g["keep"])
        per = E // G
        best = choice.view(-1, G, per).max(-1).values
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
        choice = choice.masked_fill(~kept.repeat_interleave(per, dim=1), float("-inf"))
    idx = choice.topk(top, dim=-1).indices
    sel = s.gather(1, idx)
    return idx, sel / (sel.sum(-1, keepdim=True) + 1e-20)


def moe(h: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    idx, wt = route(h, mlp["router"], w, p)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(idx[t].tolist(), wt[t]):
            a = torch.relu(w[f"{p}e{e}.up"] @ h[t]) ** 2
            out[t] += g * (w[f"{p}e{e}.down"] @ a)
    return out


# --------------------------------------------------------------------------------------- whole model
def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; `layer_outputs` collects the residual stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    pos = torch.arange(len(tokens))
    x = w["embed"][torch.tensor(tokens)]
    kv_of: Dict[int, tuple] = {}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kv_of[i] = latent_kv(x, m, w, p, eps, pos)
            c, kr = kv_of[i if m.get("kv_from") is None else int(m["kv_from"])]
            y = latent_attention(x, m, w, p, pos, c, kr)
        elif layer["type"] == "lightning":
            y, _ = lightning(x, m, w, p, eps)
        else:
            raise ValueError(layer["type"])
        x = norm_centered(alpha * x + y, w[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = norm_centered(alpha * x + moe(x, layer["mlp"], w, f"l{i}.mlp."), w[f"l{i}.norm2"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return norm_centered(x, w["final.norm"], eps) @ w["embed"].T
