"""A plain whole-sequence implementation of the Dumalix design in float64, one function per mechanism.

It shares no code with ``llmctl``: full score matrices with explicit masks, shifted sums for the
convolutions, explicit cos / sin tables.  ``cfg`` is the checkpoint's ``config.json`` as a dict,
``W`` maps the checkpoint's tensor names to tensors.  Everything runs on one sequence at a time,
positions 0 .. T-1.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x over its root mean square (eps inside the root), last dim."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), u], 0)
    y = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        y += pad[j:j + T] * w[:, j].to(F64)
    return y


def yarn_frequencies(base, dims, scaling):
    """Per-pair frequencies and the factor on cos / sin."""
    i = torch.arange(dims // 2, dtype=F64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def where(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_pairs(x, angles, amp=1.0):
    """x [..., 2n] with neighbours (2i, 2i+1) as pairs, angles [..., n]."""
    c, s = torch.cos(angles) * amp, torch.sin(angles) * amp
    a, b = x[..., 0::2], x[..., 1::2]
    return torch.stack([a * c - b * s, b * c + a * s], -1).flatten(-2)


def rotary(x, pos, rot):
    """x [T, heads, d]: the first rot['dims'] entries of every head turned by the position."""
    n = int(rot["dims"])
    f, amp = yarn_frequencies(rot["base"], n, rot.get("scaling"))
    ang = pos.to(F64)[:, None, None] * f[None, None, :]
    return torch.cat([turn_pairs(x[..., :n], ang, amp), x[..., n:]], -1)


def softmax_with_extra(s, visible, extra=None):
    """Row softmax of s [H, T, T] over the visible keys; ``extra`` [H] joins the denominator only."""
    s = s.masked_fill(~visible, float("-inf"))
    top = s.max(-1, keepdim=True).values
    if extra is not None:
        top = torch.maximum(top, extra.view(-1, 1, 1))
    e = torch.exp(s - top)
    den = e.sum(-1, keepdim=True)
    if extra is not None:
        den = den + torch.exp(extra.view(-1, 1, 1) - top)
    return e / den


def attention_mixer(h, W, p, m, eps):
    """Grouped-query attention: short convolutions, per-head norms, rotary keys and queries, turned
    values, per-head temperature, chunk mask, sink."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q, k, v = h @ W[p + "q"].to(F64).T, h @ W[p + "k"].to(F64).T, h @ W[p + "v"].to(F64).T
    if p + "q.conv" in W:
        q, k, v = causal_conv(q, W[p + "q.conv"]), causal_conv(k, W[p + "k.conv"]), causal_conv(v, W[p + "v.conv"])
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    q, k = norm_plain(q, W[p + "q.norm"], eps), norm_plain(k, W[p + "k.norm"], eps)
    q, k = rotary(q, pos, m["rot"]), rotary(k, pos, m["rot"])
    fv = float(m["rot"]["base"]) ** (-2.0 * torch.arange(dv // 2, dtype=F64) / dv)
    vang = pos.to(F64)[:, None, None] * fv[None, None, :]
    v = turn_pairs(v, vang)
    per = H // G
    k, v = k.repeat_interleave(per, 1), v.repeat_interleave(per, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"]) * W[p + "temp"].to(F64).view(H, 1, 1)
    i, j = pos[:, None], pos[None, :]
    vis = j <= i
    if m.get("mask"):
        c = int(m["mask"]["size"])
        vis = vis & (i // c == j // c)
    pr = softmax_with_extra(s, vis, W[p + "sink"].to(F64) if p + "sink" in W else None)
    o = torch.einsum("hij,jhd->ihd", pr, v)
    o = turn_pairs(o, -vang)
    return o.reshape(T, H * dv) @ W[p + "o"].to(F64).T


def latent_mixer(h, W, p, m, eps):
    """Latent attention: one normed latent and one rotary key part per token; keys and values are
    up-projections of the latent."""
    T = h.shape[0]
    H, d, dr, dv, rk = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(T)
    q = (h @ W[p + "q"].to(F64).T).view(T, H, d + dr)
    z = h @ W[p + "dkv"].to(F64).T
    c = norm_plain(z[:, :rk], W[p + "dkv.norm"], eps)
    rot = dict(m["rot"])
    k_rot = rotary(z[:, None, rk:], pos, rot)  # [T, 1, dr]
    q_rot = rotary(q[..., d:], pos, rot)
    k_un = (c @ W[p + "uk"].to(F64).T).view(T, H, d)
    v = (c @ W[p + "uv"].to(F64).T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q[..., :d], k_un) + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * float(m["scale"])
    vis = pos[None, :] <= pos[:, None]
    pr = softmax_with_extra(s, vis)
    o = torch.einsum("hij,jhd->ihd", pr, v)
    return o.reshape(T, H * dv) @ W[p + "o"].to(F64).T


def feed_forward(h, W, p, mlp):
    lim = float(mlp["limit"])
    g = (h @ W[p + "gate"].to(F64).T).clamp(max=lim)
    u = (h @ W[p + "up"].to(F64).T).clamp(-lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].to(F64).T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_mixer}


def layer(x, W, i, spec, cfg):
    eps = float(cfg["norm"]["eps"])
    p = f"l{i}."
    h = norm_one_plus(x, W[p + "norm1"], eps)
    if p + "canon1" in W:
        h = h + causal_conv(h, W[p + "canon1"])
    y = MIXERS[spec["type"]](h, W, p + "mix.", spec["mixer"], eps)
    if spec.get("mlp") is not None:
        y = y + feed_forward(norm_one_plus(x, W[p + "norm2"], eps), W, p + "mlp.", spec["mlp"])
    return x + y


def layer_order(cfg):
    """(layer index, first of a pass?) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens, trail=None):
    """Logits [T, vocab] of one sequence; ``trail`` collects the stream after every layer run."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x0 = W["embed"].to(F64)[ids]
    x = x0
    for i, first in layer_order(cfg):
        if first:
            x = torch.cat([x, x0], -1) @ W["loop.in"].to(F64).T
        x = layer(x, W, i, cfg["layers"][i], cfg)
        if trail is not None:
            trail.append(x.clone())
    x = norm_one_plus(x, W["final.norm"], float(cfg["norm"]["eps"]))
    return x @ W["head"].to(F64).T
