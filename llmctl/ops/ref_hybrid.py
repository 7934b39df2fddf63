"""CPU (fp32 torch) forms of the hybrid-mixer ops in :mod:`llmctl.ops.hybrid`.

Same signatures and cache / state layouts as the HIP kernels in ``csrc/hybrid``: the engine's
CPU path (gloo tests, no GPU) runs on these, and the kernel tests compare the HIP kernels with an
independent plain implementation, not with this file.
"""

from __future__ import annotations

from typing import Optional

import torch


def layernorm_f32(x, w, b, eps, out_dtype):
    xf = x.float()
    mu = xf.mean(-1, keepdim=True)
    var = (xf - mu).pow(2).mean(-1, keepdim=True)
    return ((xf - mu) * torch.rsqrt(var + eps) * w.float() + b.float()).to(out_dtype)


def residual_add_(x, a, b):
    x += a.float()
    if b is not None:
        x += b.float()
    return x


def rmsnorm_cols(x, w, eps, n, out_dtype):
    xf = x[:, :n].float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def _rotate(x, pos, inv_freq, dims):
    """x f32 [T, ..., n]: entries [0, dims) rotated in the rotate-half pairing."""
    half = dims // 2
    ang = pos.float()[:, None] * inv_freq.float()[None, :]  # fp32 angles
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots):
    rk = norm_w.shape[0]
    c = rmsnorm_cols(dkv, norm_w, eps, rk, torch.float32)
    kr = _rotate(dkv[:, rk:].float(), pos, inv_freq, rot_dims)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = row[ok]


def latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn):
    qr = _rotate(q[..., dn:].float(), pos, inv_freq, rot_dims)
    return torch.cat([q_lat.float(), qr], -1).to(q.dtype)


def latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk):
    """Sliding-window attention with a sink over the paged latent cache.  Sequence n owns query
    rows [cu[n], cu[n+1]); its last query sits at position ctx[n] - 1.  Keys and values are cache
    rows (value = the first ``rk`` entries of the key row), shared by all heads."""
    T, H, R = qa.shape
    bs = cache.shape[1]
    out = torch.zeros(T, H, rk, dtype=torch.float32)
    flat = cache.view(-1, R)
    cu_l, ctx_l = [int(v) for v in cu], [int(v) for v in ctx]
    for n in range(len(ctx_l)):
        a, b = cu_l[n], cu_l[n + 1]
        if b == a:
            continue
        p0 = ctx_l[n] - (b - a)  # position of the first query row
        lo = max(0, p0 - window + 1)
        kpos = torch.arange(lo, ctx_l[n])
        rows = flat[bt[n, (kpos // bs).long()].long() * bs + kpos % bs].float()  # [K, R]
        s = torch.einsum("thr,kr->htk", qa[a:b].float(), rows) * scale
        qpos = torch.arange(p0, ctx_l[n])
        d = qpos[:, None] - kpos[None, :]
        s = s.masked_fill(~((d >= 0) & (d < window)), float("-inf"))
        sk = sink.float().view(H, 1, 1)
        top = torch.maximum(s.max(-1, keepdim=True).values, sk)
        e = torch.exp(s - top)
        p = e / (e.sum(-1, keepdim=True) + torch.exp(sk - top))
        out[a:b] = torch.einsum("htk,kr->thr", p, rows[:, :rk])
    return out.to(qa.dtype)


def sigmoid_gate_mul(o, g):
    return (o.float() * torch.sigmoid(g.float())).to(g.dtype)


def mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start):
    """Token-by-token matrix-memory recurrence.  State pools S [slots, H, dk, dv], n [slots, H, dk],
    m [slots, H] (fp32) are read at ``state_slots[seq]`` (zeros when the sequence starts at
    position 0) and written back after the sequence's last token of this step."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    ig = cap * torch.tanh((if_raw[:, :H].float() + b_i.float()) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((if_raw[:, H:].float() + b_f.float()) / cap))
    cu_l = [int(x) for x in cu]
    for s in range(len(cu_l) - 1):
        a, b = cu_l[s], cu_l[s + 1]
        if a == b:
            continue
        slot = int(state_slots[s])
        if int(start[s]) == 0:
            Ss, ns, ms = torch.zeros_like(S[slot]), torch.zeros_like(n[slot]), torch.zeros_like(m[slot])
        else:
            Ss, ns, ms = S[slot].clone(), n[slot].clone(), m[slot].clone()
        for t in range(a, b):
            qt, kt, vt = q[t].float() * qscale, k[t].float(), v[t].float()
            m_new = torch.maximum(fg[t] + ms, ig[t])
            da, db = torch.exp(fg[t] + ms - m_new), torch.exp(ig[t] - m_new)
            Ss = da[:, None, None] * Ss + db[:, None, None] * kt[:, :, None] * vt[:, None, :]
            ns = da[:, None] * ns + db[:, None] * kt
            ms = m_new
            num = torch.einsum("hkv,hk->hv", Ss, qt)
            den = torch.maximum((ns * qt).sum(-1).abs(), torch.exp(-ms)) + 1e-6
            out[t] = num / den[:, None]
        S[slot], n[slot], m[slot] = Ss, ns, ms
    return out


def headnorm_gate(o, w, g, eps, out_dtype):
    T, H, dv = o.shape
    of = o.float()
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, H * dv) * w.float() * torch.sigmoid(g.float())).to(out_dtype)


def group_topk_router(logits, top, groups, keep):
    T, E = logits.shape
    s = torch.sigmoid(logits.float())
    per = E // groups
    gs = s.view(T, groups, per).topk(min(2, per), -1).values.sum(-1)
    best = gs.topk(keep, -1).indices
    ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
    ok = ok[:, :, None].expand(T, groups, per).reshape(T, E)
    idx = s.masked_fill(~ok, -1.0).topk(top, -1).indices
    return idx, s.gather(1, idx)


def swiglu_any(gu):
    f = gu.shape[-1] // 2
    g, u = gu[..., :f].float(), gu[..., f:].float()
    return (g * torch.sigmoid(g) * u).to(gu.dtype)
