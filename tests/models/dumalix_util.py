"""Helpers of the Dumalix tests: small configurations and random checkpoints written from the naming
rules of the checkpoint layout (not from the model class).  The engine, the schedule driver and the error
measure are those of the Lenitar tests."""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

from tests.models.lenitar_util import engine, rel_err, run_schedule, write_checkpoint  # noqa: F401

YARN = {"factor": 3.0, "original": 16, "fast": 4.0, "slow": 0.5}


def att(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, chunk=7, base=50.0, rot_dims=None, scaling=YARN, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "rot": {"base": base, "dims": rot_dims if rot_dims is not None else dim}, "scale": scale if scale is not None else dim ** -0.5}
    if conv:
        m["conv"] = conv
    if chunk:
        m["mask"] = {"size": chunk}
    if scaling:
        m["rot"]["scaling"] = dict(scaling)
    return {"type": "attention", "mixer": m}


def lat(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=10, base=80.0, scaling=YARN, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if scaling:
        m["rot"]["scaling"] = dict(scaling)
    return {"type": "latent_attention", "mixer": m}


def ff(n=12, limit=1.5):
    return {"kind": "dense", "ff": n, "limit": limit}


def config(layers: List[Tuple[dict, Optional[dict]]], width=20, vocab=50, eps=1e-5, taps=3, loop=None) -> dict:
    cfg = {"architecture": "Dumalix", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [dict(m, mlp=f) for m, f in layers]}
    if taps:
        cfg["canon"] = {"taps": taps}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).bfloat16().float()

    def vec(n, mean=0.0, std=1.0):
        return (mean + std * torch.randn(n, generator=g)).bfloat16().float()

    out = {"embed": vec(cfg["vocab"] * W).view(cfg["vocab"], W), "head": lin(cfg["vocab"], W), "final.norm": vec(W, 0.0, 0.2)}
    if cfg.get("loop"):
        out["loop.in"] = (lin(W, 2 * W, 0.7) + torch.cat([torch.eye(W), torch.zeros(W, W)], 1) * 0.5).bfloat16().float()
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = vec(W, 0.0, 0.2)
        if taps:
            out[p + "canon1"] = vec(W * taps, 0.0, 0.4).view(W, taps)
        q = p + "mix."
        if layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": lin(H * d, W, 2.0), q + "k": lin(G * d, W, 2.0), q + "v": lin(G * dv, W), q + "o": lin(W, H * dv),
                        q + "q.norm": vec(d, 1.0, 0.2), q + "k.norm": vec(d, 1.0, 0.2), q + "temp": vec(H, 1.5, 0.5),
                        q + "sink": vec(H, 0.0, 1.0)})
            if m.get("conv"):
                t = m["conv"]
                for n, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                    w = vec(c * t, 0.0, 0.4).view(c, t)
                    w[:, -1] += 1.0
                    out[q + n + ".conv"] = w.bfloat16().float()
        else:
            H, d, dr, dv, rk = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({q + "q": lin(H * (d + dr), W, 2.0), q + "dkv": lin(rk + dr, W, 2.0), q + "dkv.norm": vec(rk, 1.0, 0.2),
                        q + "uk": lin(H * d, rk, 2.0), q + "uv": lin(H * dv, rk), q + "o": lin(W, H * dv)})
        f = layer.get("mlp")
        if f is not None:
            out[p + "norm2"] = vec(W, 0.0, 0.2)
            out.update({p + "mlp.gate": lin(f["ff"], W, 2.0), p + "mlp.up": lin(f["ff"], W, 2.0), p + "mlp.down": lin(W, f["ff"])})
    return out
