"""Ops of the hybrid sequence mixers: latent attention (compressed K/V cache, sliding window,
softmax sink), the mLSTM matrix memory, the group-limited sigmoid router, and the fp32 residual
stream of parallel layers.

GPU tensors run the HIP kernels of ``csrc/hybrid`` (``torch.ops.llmctl_hybrid.*``, library
``_llmctl_hybrid.so``); CPU tensors run :mod:`llmctl.ops.ref_hybrid`.  All activations are
token-major ``[T, features]`` over the step's packed tokens; sequences are described by ``cu``
(row offsets, int32 [n + 1]), ``ctx`` (context length after the step, int32 [n]) and block tables.

Precision: norms, rotary angles, attention scores / softmax, the recurrence with its gates and the
residual stream are fp32 inside every kernel whatever the activation dtype (bf16 or fp32).
"""

from __future__ import annotations

import torch

from . import ref_hybrid as ref
from ._lib import native_hybrid, use_native


def layernorm_f32(x, w, b, eps: float, out_dtype):
    """LayerNorm of the fp32 residual stream ``x [T, W]`` -> ``out_dtype``."""
    if use_native(x):
        return native_hybrid().layernorm_f32(x, w, b, eps, out_dtype == torch.bfloat16)
    return ref.layernorm_f32(x, w, b, eps, out_dtype)


def residual_add_(x, a, b=None):
    """``x += a (+ b)`` on the fp32 residual stream (a, b: any float dtype)."""
    if use_native(x):
        native_hybrid().residual_add_(x, a, b)
        return x
    return ref.residual_add_(x, a, b)


def add_layernorm_f32_(x, a, b, w, bias, eps: float, out_dtype):
    """``x += a (+ b)`` in place, then LayerNorm(x) -> ``out_dtype``: the parallel layer's residual
    update and the next layer's norm in one pass over the stream."""
    if use_native(x):
        return native_hybrid().add_layernorm_f32_(x, a, b, w, bias, eps, out_dtype == torch.bfloat16)
    ref.residual_add_(x, a, b)
    return ref.layernorm_f32(x, w, bias, eps, out_dtype)


def rmsnorm_cols(x, w, eps: float, n: int, out_dtype):
    """RMS norm (weight ``w [n]``) of the first ``n`` columns of ``x [T, N]`` -> ``[T, n]``."""
    if use_native(x):
        return native_hybrid().rmsnorm_cols(x, w, eps, n, out_dtype == torch.bfloat16)
    return ref.rmsnorm_cols(x, w, eps, n, out_dtype)


def latent_kv_write(dkv, norm_w, eps: float, pos, inv_freq, rot_dims: int, cache, slots):
    """The down-projected K/V row ``dkv [T, rank + rot]``: RMS norm of the latent part, rotary on
    the shared key part, both written to the paged cache row ``[rank | rot]`` at ``slots``."""
    if use_native(dkv):
        native_hybrid().latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots)
    else:
        ref.latent_kv_write(dkv, norm_w, eps, pos, inv_freq, rot_dims, cache, slots)


def latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims: int, dn: int):
    """Query rows in the cache's layout: ``[q_lat | rotary(q[..., dn:])]`` per head, where ``q_lat
    [T, H, rank]`` is the unrotated query part carried into the latent space (q W_uk)."""
    if use_native(q):
        return native_hybrid().latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn)
    return ref.latent_q_assemble(q_lat, q, pos, inv_freq, rot_dims, dn)


def latent_attention_prefill(qa, cache, bt, cu, ctx, window: int, sink, scale: float, rk: int, max_q: int,
                             mfma: bool = True):
    """Prompt portions: sequence n's query rows ``[cu[n], cu[n+1])`` end at position ``ctx[n]-1``;
    ``max_q``: the longest portion (sizes the launch).  bf16 shapes that fit run on the matrix cores
    (``mfma=False`` forces the generic fp32-SIMT kernel, which also serves fp32)."""
    if use_native(qa):
        return native_hybrid().latent_attn_prefill(qa, cache, bt, cu, ctx, window, sink, scale, rk, max_q, mfma)
    return ref.latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk)


def latent_attention_decode(qa, cache, bt, ctx, window: int, sink, scale: float, rk: int, mfma: bool = True):
    """One query row per sequence, at position ``ctx[n] - 1``."""
    if use_native(qa):
        return native_hybrid().latent_attn_decode(qa, cache, bt, ctx, window, sink, scale, rk, mfma)
    cu = torch.arange(qa.shape[0] + 1, dtype=torch.int32)
    return ref.latent_attention(qa, cache, bt, cu, ctx, window, sink, scale, rk)


def sigmoid_gate_mul(o, g):
    """``o * sigmoid(g)`` -> g's dtype."""
    if use_native(g):
        return native_hybrid().sigmoid_gate_mul(o, g)
    return ref.sigmoid_gate_mul(o, g)


def mlstm_scan(q, k, v, if_raw, b_i, b_f, cap: float, qscale: float, S, n, m, state_slots, cu, start, slab: bool = False):
    """mLSTM recurrence over the step's tokens; returns the un-normalised head outputs fp32
    ``[T, H, dv]`` and updates the state pools in place.  ``slab`` forces the block-per-tile kernel
    (the form for key dims above 128) where the wave-per-tile one would run."""
    if use_native(q):
        return native_hybrid().mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start, slab)
    return ref.mlstm_scan(q, k, v, if_raw, b_i, b_f, cap, qscale, S, n, m, state_slots, cu, start)


def headnorm_gate(o, w, g, eps: float, out_dtype):
    """Per-head unit-RMS of ``o [T, H, dv]`` (fp32), times ``w [H*dv]``, times ``sigmoid(g)``."""
    if use_native(o):
        return native_hybrid().headnorm_gate(o, w, g, eps, out_dtype == torch.bfloat16)
    return ref.headnorm_gate(o, w, g, eps, out_dtype)


def group_topk_router(logits, top: int, groups: int, keep: int):
    """Sigmoid scores of ``logits [T, E]`` (fp32); experts in ``groups`` equal groups of neighbours,
    a group scored by the sum of its two best experts, the ``top`` best experts of the ``keep`` best
    groups chosen.  Returns (expert ids int64 [T, top], their scores fp32 [T, top])."""
    if use_native(logits):
        return native_hybrid().group_topk_router(logits, top, groups, keep)
    return ref.group_topk_router(logits, top, groups, keep)


def swiglu_any(gu):
    """``silu(gate) * up`` of ``gu [..., 2F]`` = ``[gate | up]``, bf16 or fp32."""
    if use_native(gu):
        return native_hybrid().swiglu_any(gu.contiguous())
    return ref.swiglu_any(gu)
