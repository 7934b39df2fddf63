"""Sequence mixers beside softmax attention, for serving steps over packed tokens.

* :class:`LatentAttention` — attention whose keys and values are up-projections of one small
  latent per token; only the latent and one rotary key part shared by all heads are cached.  With
  ``k = W_uk c`` the score ``q . k`` equals ``(W_uk^T q) . c``, so the step carries the query into the
  latent space once and attends the cache rows directly (one "head" of width ``rank + rot`` serves all
  query heads), and the value up-projection is applied to the attended latent afterwards.  Options:
  sliding window, a per-head softmax sink, a sigmoid output gate, a low-rank query path.
* :class:`MLSTM` — the xLSTM matrix memory: per head a ``[dk, dv]`` state with exponential input gate,
  sigmoid forget gate (both soft-capped) and a running log-scale stabiliser; state lives in a slot
  pool of the engine's cache, one slot per live sequence.

Both read a :class:`StepBatch` (the engine's description of one step: packed prompt portions first,
then one row per decoding sequence) and the layer's part of the engine's cache.  Projections are
vendor GEMMs on fused weights; everything else is a kernel of :mod:`llmctl.ops.hybrid`.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from llmctl.ops import hybrid as hops


@dataclass
class StepBatch:
    """One engine step over T packed tokens: rows [0, Tp) are prompt portions of ``len(p_ctx)``
    sequences (row offsets ``p_cu``), rows [Tp, T) one decoded token each."""
    ids: torch.Tensor  # int64 [T]
    pos: torch.Tensor  # int32 [T]
    slots: torch.Tensor  # int64 [T] cache slot of every token (block * block_size + offset)
    Tp: int
    p_cu: Optional[torch.Tensor]  # int32 [np + 1]
    p_ctx: Optional[torch.Tensor]  # int32 [np] context length after the step
    p_bt: Optional[torch.Tensor]  # int32 [np, max_blocks]
    d_ctx: Optional[torch.Tensor]  # int32 [nd]
    d_bt: Optional[torch.Tensor]  # int32 [nd, max_blocks]
    # all sequences (portions, then decodes): row offsets, first position, recurrent-state slot
    cu: torch.Tensor  # int32 [n + 1]
    start: torch.Tensor  # int32 [n]
    state: torch.Tensor  # int32 [n]
    max_q: int = 0  # the longest prompt portion of the step
    cu_host: Optional[list] = None  # ``cu`` on the host (chunk-parallel scans split long portions)


def _init(t: torch.Tensor, std: float) -> None:
    with torch.no_grad():
        t.normal_(0.0, std)


class LatentAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, q_rank: int,
                 rot_base: float, rot_dims: int, scale: float, window: int, eps: float, device=None, dtype=None):
        super().__init__()
        self.width, self.H, self.dn, self.dr, self.dv = width, heads, dim, rot_dim, vdim
        self.rk, self.qr, self.rot_dims, self.scale, self.window, self.eps = kv_rank, q_rank, rot_dims, scale, window, eps
        if rot_dims > rot_dim or rot_dims % 2:
            raise ValueError("rotary dims must be even and fit the rotated part")
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        # one GEMM for everything that reads the layer input: [W_dq ; W_dkv ; W_g]
        self.w_in = nn.Parameter(torch.empty(q_rank + kv_rank + rot_dim + heads * vdim, width, **kw))
        self.w_uq = nn.Parameter(torch.empty(heads * (dim + rot_dim), q_rank, **kw))
        self.w_uk = nn.Parameter(torch.empty(heads, dim, kv_rank, **kw))  # per head [dn, rank]
        self.w_uv = nn.Parameter(torch.empty(heads, vdim, kv_rank, **kw))  # per head [dv, rank]
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        self.q_norm = nn.Parameter(torch.ones(q_rank, **f32))
        self.kv_norm = nn.Parameter(torch.ones(kv_rank, **f32))
        self.sink = nn.Parameter(torch.zeros(heads, **f32))
        for w in (self.w_in, self.w_uq, self.w_uk, self.w_uv, self.w_o):
            _init(w, 0.02)
        i = torch.arange(rot_dims // 2, dtype=torch.float64)
        self.register_buffer("inv_freq", (float(rot_base) ** (-2.0 * i / rot_dims)).to(torch.float32).to(device),
                             persistent=False)

    cache_kind = "latent"

    @property
    def cache_row(self) -> int:
        return self.rk + self.dr

    def step(self, h: torch.Tensor, b: StepBatch, cache: torch.Tensor) -> torch.Tensor:
        T, H = h.shape[0], self.H
        z = F.linear(h, self.w_in)
        a, c = self.qr, self.qr + self.rk + self.dr
        hops.latent_kv_write(z[:, a:c], self.kv_norm, self.eps, b.pos, self.inv_freq, self.rot_dims, cache, b.slots)
        cq = hops.rmsnorm_cols(z[:, :a], self.q_norm, self.eps, self.qr, h.dtype)
        q = F.linear(cq, self.w_uq).view(T, H, self.dn + self.dr)
        q_lat = torch.bmm(q[:, :, :self.dn].transpose(0, 1), self.w_uk).transpose(0, 1)  # [T, H, rank]
        qa = hops.latent_q_assemble(q_lat, q, b.pos, self.inv_freq, self.rot_dims, self.dn)
        outs = []
        if b.Tp:
            outs.append(hops.latent_attention_prefill(qa[:b.Tp], cache, b.p_bt, b.p_cu, b.p_ctx, self.window,
                                                      self.sink, self.scale, self.rk, b.max_q))
        if T > b.Tp:
            outs.append(hops.latent_attention_decode(qa[b.Tp:], cache, b.d_bt, b.d_ctx, self.window, self.sink,
                                                     self.scale, self.rk))
        o_lat = outs[0] if len(outs) == 1 else torch.cat(outs)
        o = torch.bmm(o_lat.transpose(0, 1), self.w_uv.transpose(1, 2)).transpose(0, 1).reshape(T, H * self.dv)
        return F.linear(hops.sigmoid_gate_mul(o, z[:, c:]), self.w_o)


class MLSTM(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, device=None,
                 dtype=None):
        super().__init__()
        self.width, self.H, self.dk, self.dv, self.cap, self.eps = width, heads, dim, vdim, float(gate_cap), eps
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        # [W_q ; W_k ; W_v ; W_g] in one GEMM; the two gate rows per head stay fp32
        self.w_in = nn.Parameter(torch.empty(2 * heads * dim + 2 * heads * vdim, width, **kw))
        self.w_if = nn.Parameter(torch.empty(2 * heads, width, **f32))
        self.b_i = nn.Parameter(torch.zeros(heads, **f32))
        self.b_f = nn.Parameter(torch.full((heads,), 3.0, **f32))
        self.norm = nn.Parameter(torch.ones(heads * vdim, **f32))
        self.w_o = nn.Parameter(torch.empty(width, heads * vdim, **kw))
        for w in (self.w_in, self.w_if, self.w_o):
            _init(w, 0.02)

    cache_kind = "state"

    def state_shapes(self):
        return [(self.H, self.dk, self.dv), (self.H, self.dk), (self.H,)]

    def step(self, h: torch.Tensor, b: StepBatch, state) -> torch.Tensor:
        T, H, dk, dv = h.shape[0], self.H, self.dk, self.dv
        z = F.linear(h, self.w_in)
        q, k = z[:, :H * dk].view(T, H, dk), z[:, H * dk:2 * H * dk].view(T, H, dk)
        v = z[:, 2 * H * dk:2 * H * dk + H * dv].view(T, H, dv)
        g = z[:, 2 * H * dk + H * dv:]
        gates = F.linear(h.float(), self.w_if)  # fp32 [T, 2H]
        S, n, m = state
        o = hops.mlstm_scan(q, k, v, gates, self.b_i, self.b_f, self.cap, 1.0 / math.sqrt(dk), S, n, m, b.state,
                            b.cu, b.start, cu_host=b.cu_host)
        return F.linear(hops.headnorm_gate(o, self.norm, g, self.eps, h.dtype), self.w_o)
