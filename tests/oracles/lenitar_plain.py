"""Plain whole-sequence implementation of the Lenitar design, one function per mechanism.

Everything is float64 torch on the CPU, written from the design's equations with no code
shared with ``llmctl``: full score matrices with explicit masks, a token loop for the
recurrence, a per-token loop for the routed experts.  It is the yardstick the kernel and
engine tests compare against; it is slow on purpose.

Weights are a ``dict`` name -> tensor with the checkpoint's names (``l<i>.mix.dq`` ...);
``cfg`` is the parsed ``config.json``.
"""

from __future__ import annotations

import math
from typing import Dict, List, Tuple

import torch

F64 = torch.float64


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate_half(x, pos, base: float, dims: int):
    """x [T, ..., n]: the first ``dims`` entries of the last axis are rotated, entry i with
    entry i + dims/2, by the angle pos * base^(-2i/dims)."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    ang = pos.to(F64)[:, None] * base ** (-2.0 * i / dims)  # [T, half]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_attention(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    """h [T, width] -> [T, width]; positions are 0..T-1."""
    T = h.shape[0]
    H, dn, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = unit_rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).view(T, H, dn + dr)
    q_plain, q_rot = q[..., :dn], rotate_half(q[..., dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    dkv = h @ W[p + "dkv"].T
    c = unit_rms(dkv[:, :rk], eps) * W[p + "dkv.norm"]
    k_rot = rotate_half(dkv[:, rk:], pos, m["rot"]["base"], m["rot"]["dims"])  # [T, dr], shared by heads
    k_plain = (c @ W[p + "uk"].T).view(T, H, dn)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < m["mask"]["size"])
    s = s.masked_fill(~seen, -math.inf)
    sink = W[p + "sink"].to(F64).view(H, 1, 1)
    top = torch.maximum(s.max(-1, keepdim=True).values, sink)
    e = torch.exp(s - top)
    wgt = e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))
    o = torch.einsum("hij,jhd->ihd", wgt, v).reshape(T, H * dv)
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def mlstm(h, W: Dict[str, torch.Tensor], p: str, m: dict, eps: float):
    T = h.shape[0]
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ W[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, dk)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    S = torch.zeros(H, dk, dv, dtype=F64)
    n = torch.zeros(H, dk, dtype=F64)
    mx = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        a, b = torch.exp(fg[t] + mx - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hkv,hk->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    o = unit_rms(out, eps).reshape(T, H * dv) * W[p + "norm"]
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def route(h, w_router, r: dict) -> Tuple[torch.Tensor, torch.Tensor]:
    """Chosen experts [T, top] and their weights [T, top]."""
    E, top, G, keep = r["experts"], r["top"], r["groups"]["count"], r["groups"]["keep"]
    s = torch.sigmoid(h @ w_router.T)  # [T, E]
    per = E // G
    gs = s.view(-1, G, per).topk(min(2, per), -1).values.sum(-1)  # [T, G]
    best = gs.topk(keep, -1).indices
    allowed = torch.zeros(s.shape[0], G, dtype=torch.bool).scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(-1, -1, per).reshape(-1, E)
    idx = s.masked_fill(~allowed, -1.0).topk(top, -1).indices
    return idx, s.gather(1, idx)


def moe(h, W: Dict[str, torch.Tensor], p: str, f: dict):
    idx, wgt = route(h, W[p + "router"], f["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wgt[t]):
            g = W[f"{p}e{e}.gate"] @ h[t]
            u = W[f"{p}e{e}.up"] @ h[t]
            out[t] += w * (W[f"{p}e{e}.down"] @ (g * torch.sigmoid(g) * u))
    return out


MIXERS = {"latent_attention": latent_attention, "mlstm": mlstm}


def forward(tokens: List[int], W: Dict[str, torch.Tensor], cfg: dict):
    """Logits [T, vocab] and the residual stream after every layer [L, T, width]."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    trail = []
    for li, layer in enumerate(cfg["layers"]):
        p = f"l{li}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        y = MIXERS[layer["type"]](h, W, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            y = y + moe(h, W, p + "mlp.", layer["mlp"])
        x = x + y
        trail.append(x)
    xn = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return xn @ W["head"].T, torch.stack(trail)
