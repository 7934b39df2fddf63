"""Lenitar: a decoder-only hybrid — parallel layers (one LayerNorm feeding a sequence mixer and a
routed feed-forward, both added to the residual), mixers chosen per layer between latent attention
and the mLSTM matrix memory (:mod:`llmctl.models.mixers`), group-limited sigmoid-routed experts
(:class:`llmctl.models.moe.GroupLimitedMoE`), scaled embedding, LayerNorm before the head.

Checkpoint layout: ``config.json`` (``architecture``, ``vocab``, ``width``, ``embedding.scale``,
``norm.eps``, ``layers`` = one entry per layer with ``type``, ``mixer`` sizes and ``mlp`` or null)
and ``model.safetensors`` with tensors ``embed``, ``l<i>.norm1[.b]``, ``l<i>.mix.*``,
``l<i>.mlp.router``, ``l<i>.mlp.e<j>.{gate,up,down}``, ``final.norm[.b]``, ``head``; linear weights
``[out, in]``.  Every size is read from the config; layers may differ from one another.

The residual stream is fp32 whatever the activation dtype; norms, rotary angles, attention softmax,
gates and the recurrence are fp32 inside the kernels.
"""

from __future__ import annotations

import copy
import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from llmctl.ops import hybrid as hops

from .mixers import MLSTM, LatentAttention, StepBatch
from .moe import GroupLimitedMoE

ARCHITECTURE = "Lenitar"


@dataclass
class LenitarConfig:
    name: str = "lenitar"
    architecture: str = ARCHITECTURE
    vocab_size: int = 512
    hidden: int = 256
    layer_specs: List[Dict[str, Any]] = field(default_factory=list)
    layer_norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    max_position_embeddings: int = 8192
    extra: Dict[str, Any] = field(default_factory=dict)

    # what the serving engine asks of any model config
    is_moe = True  # routed experts size their segments on the host: eager steps, no captured graphs
    tie_word_embeddings = False

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LenitarConfig":
        d = copy.deepcopy(dict(d))
        kw = dict(architecture=d.pop("architecture", ARCHITECTURE), vocab_size=int(d.pop("vocab")),
                  hidden=int(d.pop("width")), layer_specs=list(d.pop("layers")),
                  layer_norm_eps=float(d.pop("norm")["eps"]),
                  embedding_scale=float((d.pop("embedding", None) or {}).get("scale", 1.0)))
        if "name" in d:
            kw["name"] = d.pop("name")
        if "max_position_embeddings" in d:
            kw["max_position_embeddings"] = int(d.pop("max_position_embeddings"))
        for spec in kw["layer_specs"]:
            if spec["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown mixer type {spec['type']!r} (known: {sorted(MIXER_TYPES)})")
            mlp = spec.get("mlp")
            if mlp is not None and mlp.get("kind", "moe") != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        return cls(extra=d, **kw)

    @classmethod
    def from_file(cls, path) -> "LenitarConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architecture, "name": self.name, "vocab": self.vocab_size, "width": self.hidden,
             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.layer_norm_eps},
             "layers": copy.deepcopy(self.layer_specs), "max_position_embeddings": self.max_position_embeddings}
        d.update(self.extra)
        return d

    def num_parameters(self, include_embedding: bool = True) -> int:
        with torch.device("meta"):
            m = LenitarLM(self, dtype=torch.bfloat16)
        n = sum(p.numel() for p in m.parameters())
        return n if include_embedding else n - 2 * self.vocab_size * self.hidden


def _latent(width, m, eps, **kw):
    rot = m.get("rot") or {}
    return LatentAttention(width, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                           vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]),
                           rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", m["rot_dim"])),
                           scale=float(m["scale"]), window=int(m["mask"]["size"]), eps=eps, **kw)


def _mlstm(width, m, eps, **kw):
    return MLSTM(width, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), gate_cap=float(m["gate_cap"]),
                 eps=eps, **kw)


MIXER_TYPES = {"latent_attention": _latent, "mlstm": _mlstm}


class LenitarLayer(nn.Module):
    def __init__(self, cfg: LenitarConfig, spec: Dict[str, Any], device=None, dtype=None):
        super().__init__()
        W = cfg.hidden
        f32 = dict(device=device, dtype=torch.float32)
        self.norm_w = nn.Parameter(torch.ones(W, **f32))
        self.norm_b = nn.Parameter(torch.zeros(W, **f32))
        self.mixer = MIXER_TYPES[spec["type"]](W, spec["mixer"], cfg.layer_norm_eps, device=device, dtype=dtype)
        mlp = spec.get("mlp")
        self.ff = None
        if mlp is not None:
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            self.ff = GroupLimitedMoE(W, int(mlp["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(g["count"]),
                                      int(g["keep"]), device=device, dtype=dtype)


class LenitarLM(nn.Module):
    is_hybrid = True

    def __init__(self, cfg: LenitarConfig, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        kw = dict(device=device, dtype=dtype)
        f32 = dict(device=device, dtype=torch.float32)
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden, **kw))
        self.layers = nn.ModuleList([LenitarLayer(cfg, s, **kw) for s in cfg.layer_specs])
        self.final_norm_w = nn.Parameter(torch.ones(cfg.hidden, **f32))
        self.final_norm_b = nn.Parameter(torch.zeros(cfg.hidden, **f32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, cfg.hidden, **kw))
        with torch.no_grad():
            self.embed.normal_(0.0, 0.02)
            self.lm_head.normal_(0.0, 0.02)

    @property
    def dtype(self):
        return self.embed.dtype

    @property
    def has_recurrent_state(self) -> bool:
        return any(l.mixer.cache_kind == "state" for l in self.layers)

    def head_weight(self):
        return self.lm_head

    # ------------------------------------------------------------------ serving step
    def step(self, b: StepBatch, cache, rows: Optional[torch.Tensor] = None, trail: Optional[list] = None):
        """Run the step's packed tokens through all layers against the engine's cache (``cache.layer(i)``:
        the paged latent pool or the state pools of layer i).  Returns the fp32 residual stream of
        ``rows`` (all rows if None) after the last layer; ``trail`` collects it after every layer."""
        cfg, eps, dt = self.cfg, self.cfg.layer_norm_eps, self.dtype
        x = F.embedding(b.ids, self.embed).float() * cfg.embedding_scale  # fp32 residual stream
        h = hops.layernorm_f32(x, self.layers[0].norm_w, self.layers[0].norm_b, eps, dt)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            y = layer.mixer.step(h, b, cache.layer(i))
            z = layer.ff(h) if layer.ff is not None else None
            if i + 1 < n and trail is None:
                nxt = self.layers[i + 1]
                h = hops.add_layernorm_f32_(x, y, z, nxt.norm_w, nxt.norm_b, eps, dt)
            else:
                hops.residual_add_(x, y, z)
                if trail is not None:
                    trail.append(x.clone())
                    if i + 1 < n:
                        h = hops.layernorm_f32(x, self.layers[i + 1].norm_w, self.layers[i + 1].norm_b, eps, dt)
        return x if rows is None else x.index_select(0, rows)

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        xn = hops.layernorm_f32(x.contiguous(), self.final_norm_w, self.final_norm_b, self.cfg.layer_norm_eps,
                                self.dtype)
        return F.linear(xn, self.lm_head)

    # ------------------------------------------------------------------ checkpoint names
    @torch.no_grad()
    def load_named(self, W: Dict[str, torch.Tensor]) -> None:
        """Copy a checkpoint's tensors (its names, see the module docstring) into the fused parameters."""
        def put(dst, src):
            if tuple(dst.shape) != tuple(src.shape):
                raise ValueError(f"shape {tuple(src.shape)} does not fit {tuple(dst.shape)}")
            dst.copy_(src.to(dst.dtype))

        put(self.embed, W["embed"])
        put(self.lm_head, W["head"])
        put(self.final_norm_w, W["final.norm"])
        put(self.final_norm_b, W["final.norm.b"])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm_w, W[p + "norm1"])
            put(layer.norm_b, W[p + "norm1.b"])
            m, q = layer.mixer, p + "mix."
            if isinstance(m, LatentAttention):
                put(m.w_in, torch.cat([W[q + "dq"], W[q + "dkv"], W[q + "g"]], 0))
                put(m.q_norm, W[q + "dq.norm"])
                put(m.kv_norm, W[q + "dkv.norm"])
                put(m.w_uq, W[q + "uq"])
                put(m.w_uk.view(m.H * m.dn, m.rk), W[q + "uk"])
                put(m.w_uv.view(m.H * m.dv, m.rk), W[q + "uv"])
                put(m.sink, W[q + "sink"])
                put(m.w_o, W[q + "o"])
            else:
                put(m.w_in, torch.cat([W[q + "q"], W[q + "k"], W[q + "v"], W[q + "g"]], 0))
                put(m.w_if, torch.cat([W[q + "i"], W[q + "f"]], 0))
                put(m.b_i, W[q + "i.b"])
                put(m.b_f, W[q + "f.b"])
                put(m.norm, W[q + "norm"])
                put(m.w_o, W[q + "o"])
            if layer.ff is not None:
                f = p + "mlp."
                put(layer.ff.w_router, W[f + "router"])
                for e in range(layer.ff.E):
                    put(layer.ff.experts_up[e], torch.cat([W[f"{f}e{e}.gate"], W[f"{f}e{e}.up"]], 0))
                    put(layer.ff.experts_down[e], W[f"{f}e{e}.down"])

    @torch.no_grad()
    def export_named(self) -> Dict[str, torch.Tensor]:
        """The inverse of :meth:`load_named`: tensors under the checkpoint's names."""
        out = {"embed": self.embed, "head": self.lm_head, "final.norm": self.final_norm_w,
               "final.norm.b": self.final_norm_b}
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"], out[p + "norm1.b"] = layer.norm_w, layer.norm_b
            m, q = layer.mixer, p + "mix."
            if isinstance(m, LatentAttention):
                a, c = m.qr, m.qr + m.rk + m.dr
                out.update({q + "dq": m.w_in[:a], q + "dkv": m.w_in[a:c], q + "g": m.w_in[c:], q + "dq.norm": m.q_norm,
                            q + "dkv.norm": m.kv_norm, q + "uq": m.w_uq, q + "uk": m.w_uk.reshape(m.H * m.dn, m.rk),
                            q + "uv": m.w_uv.reshape(m.H * m.dv, m.rk), q + "sink": m.sink, q + "o": m.w_o})
            else:
                a, c = m.H * m.dk, 2 * m.H * m.dk + m.H * m.dv
                out.update({q + "q": m.w_in[:a], q + "k": m.w_in[a:2 * a], q + "v": m.w_in[2 * a:c], q + "g": m.w_in[c:],
                            q + "i": m.w_if[:m.H], q + "f": m.w_if[m.H:], q + "i.b": m.b_i, q + "f.b": m.b_f,
                            q + "norm": m.norm, q + "o": m.w_o})
            if layer.ff is not None:
                f, ff = p + "mlp.", layer.ff.ff
                out[f + "router"] = layer.ff.w_router
                for e in range(layer.ff.E):
                    out[f"{f}e{e}.gate"], out[f"{f}e{e}.up"] = layer.ff.experts_up[e][:ff], layer.ff.experts_up[e][ff:]
                    out[f"{f}e{e}.down"] = layer.ff.experts_down[e]
        return {k: v.detach().clone().contiguous() for k, v in out.items()}


def load_lenitar(ck: Path, cfg: LenitarConfig, device=None, dtype=torch.bfloat16) -> LenitarLM:
    from safetensors import safe_open

    model = LenitarLM(cfg, device=device, dtype=dtype)
    with safe_open(str(ck / "model.safetensors"), framework="pt", device="cpu") as f:
        W = {k: f.get_tensor(k) for k in f.keys()}
    model.load_named(W)
    return model


def lenitar_template(width: int = 256, layers: int = 4, heads: int = 4, vocab: int = 512, every: int = 4,
                     experts: int = 8, top: int = 2, groups: int = 2, keep: int = 1, ff: int = 128,
                     window: int = 128) -> LenitarConfig:
    """A random-init configuration for benchmarks and smoke runs: latent attention in every layer but
    each ``every``-th, which is an mLSTM; sizes scale with ``width`` and ``heads``."""
    d = width // heads
    att = {"heads": heads, "dim": d, "rot_dim": max(d // 2, 2) // 2 * 2, "vdim": d, "kv_rank": max(width // 4, 8),
           "q_rank": max(width // 2, 8), "rot": {"base": 10000.0, "dims": max(d // 2, 2) // 2 * 2},
           "scale": (d + max(d // 2, 2) // 2 * 2) ** -0.5, "mask": {"size": window}}
    rec = {"heads": heads, "dim": d // 2 if d >= 4 else d, "vdim": d, "gate_cap": 15.0}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top,
                                                            "groups": {"count": groups, "keep": keep}}}
    specs = [{"type": "mlstm" if (i + 1) % every == 0 else "latent_attention",
              "mixer": copy.deepcopy(rec if (i + 1) % every == 0 else att), "mlp": copy.deepcopy(mlp)}
             for i in range(layers)]
    return LenitarConfig(name=f"lenitar-w{width}-l{layers}", vocab_size=vocab, hidden=width, layer_specs=specs,
                         layer_norm_eps=1e-6, embedding_scale=float(width) ** 0.5)
