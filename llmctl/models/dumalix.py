"""Dumalix: a decoder-only design of parallel layers with a looped middle.

* A layer reads the fp32 residual stream x through two RMS norms (weights stored around zero, applied
  as ``1 + w``; both norms share one statistic) and adds both branches: ``x += mixer(conv(norm1(x))) +
  ff(norm2(x))``.  ``conv`` is a short causal convolution over time added to its input
  (:class:`llmctl.models.mixers.CausalConv`, residual form); its last inputs are per-sequence state.
* Mixers, chosen per layer: ``attention`` = :class:`~llmctl.models.mixers.GroupedAttention` (short
  convolutions on q / k / v, per-head q / k norms, YaRN rotary on neighbour pairs, values turned by
  their position and turned back on the output, per-head temperature, chunked mask, softmax sink) and
  ``latent_attention`` = :class:`~llmctl.models.mixers.LatentAttention` (full-rank query, causal, no
  sink or gate, YaRN rotary on the shared key part).
* Feed-forward: :class:`~llmctl.models.mixers.ClampedGLU`.
* ``loop`` = ``{start, stop, times}``: layers ``start .. stop-1`` run ``times`` times in a row with the
  same weights; every pass keeps its own cache rows and state, and begins with ``x <- W_in [x ; x0]``
  (x0 = the embedding output).  The cache therefore has one entry per layer *run*.

Checkpoint layout: ``config.json`` (``architecture``, ``vocab``, ``width``, ``norm.eps``, ``canon.taps``,
``loop``, ``layers`` = one entry per layer with ``type``, ``mixer`` and ``mlp`` or null) and
``model.safetensors`` with ``embed``, ``loop.in``, ``l<i>.norm1|norm2|canon1``, ``l<i>.mix.*``,
``l<i>.mlp.{gate,up,down}``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""

from __future__ import annotations

import copy
import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from llmctl.ops import hybrid as hops

from .mixers import CausalConv, ClampedGLU, GroupedAttention, LatentAttention, StepBatch

ARCHITECTURE = "Dumalix"


@dataclass
class DumalixConfig:
    name: str = "dumalix"
    architecture: str = ARCHITECTURE
    vocab_size: int = 512
    hidden: int = 256
    layer_specs: List[Dict[str, Any]] = field(default_factory=list)
    layer_norm_eps: float = 1e-5
    canon_taps: int = 0  # taps of the convolution on the mixer's input; 0 = none
    loop: Optional[Dict[str, int]] = None  # {"start", "stop", "times"}
    max_position_embeddings: int = 8192
    extra: Dict[str, Any] = field(default_factory=dict)

    is_moe = False
    tie_word_embeddings = False

    @property
    def layers(self) -> int:
        return len(self.layer_specs)

    def runs(self) -> List[Tuple[int, bool]]:
        """(layer, first of a loop pass?) for every layer run, in order."""
        n = len(self.layer_specs)
        if not self.loop:
            return [(i, False) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        if not (0 <= a <= b <= n) or times < 0:
            raise ValueError(f"loop {self.loop} does not fit {n} layers")
        out = [(i, False) for i in range(a)]
        for _ in range(times):
            out += [(i, i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "DumalixConfig":
        d = copy.deepcopy(dict(d))
        kw = dict(architecture=d.pop("architecture", ARCHITECTURE), vocab_size=int(d.pop("vocab")),
                  hidden=int(d.pop("width")), layer_specs=list(d.pop("layers")),
                  layer_norm_eps=float(d.pop("norm")["eps"]),
                  canon_taps=int((d.pop("canon", None) or {}).get("taps", 0)), loop=d.pop("loop", None))
        for k in ("name", "max_position_embeddings"):
            if k in d:
                kw[k] = d.pop(k)
        for spec in kw["layer_specs"]:
            if spec["type"] not in MIXER_TYPES:
                raise ValueError(f"unknown mixer type {spec['type']!r} (known: {sorted(MIXER_TYPES)})")
            mlp = spec.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
        cfg = cls(extra=d, **kw)
        cfg.runs()
        return cfg

    @classmethod
    def from_file(cls, path) -> "DumalixConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def to_dict(self) -> Dict[str, Any]:
        d = {"architecture": self.architecture, "name": self.name, "vocab": self.vocab_size, "width": self.hidden,
             "norm": {"eps": self.layer_norm_eps}, "layers": copy.deepcopy(self.layer_specs),
             "max_position_embeddings": self.max_position_embeddings}
        if self.canon_taps:
            d["canon"] = {"taps": self.canon_taps}
        if self.loop:
            d["loop"] = dict(self.loop)
        d.update(self.extra)
        return d

    def num_parameters(self, include_embedding: bool = True) -> int:
        with torch.device("meta"):
            m = DumalixLM(self, dtype=torch.bfloat16)
        n = sum(p.numel() for p in m.parameters())
        return n if include_embedding else n - 2 * self.vocab_size * self.hidden


def _attention(width, m, eps, **kw):
    rot = m["rot"]
    return GroupedAttention(width, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                            vdim=int(m["vdim"]), rot_base=float(rot["base"]), rot_dims=int(rot.get("dims", m["dim"])),
                            scale=float(m["scale"]), eps=eps, conv_taps=int(m.get("conv") or 0),
                            rot_scaling=rot.get("scaling"), interleaved=True, rotate_values=True, temperature=True,
                            chunk=(m.get("mask") or {}).get("size"), sink=True, **kw)


def _latent(width, m, eps, **kw):
    rot = m["rot"]
    return LatentAttention(width, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                           kv_rank=int(m["kv_rank"]), q_rank=None, rot_base=float(rot["base"]),
                           rot_dims=int(rot.get("dims", m["rot_dim"])), scale=float(m["scale"]), window=None, eps=eps,
                           sink=False, gate=False, rot_scaling=rot.get("scaling"), interleaved=True, **kw)


MIXER_TYPES = {"attention": _attention, "latent_attention": _latent}


class DumalixLayer(nn.Module):
    def __init__(self, cfg: DumalixConfig, spec: Dict[str, Any], device=None, dtype=None):
        super().__init__()
        W = cfg.hidden
        f32 = dict(device=device, dtype=torch.float32)
        self.norm1 = nn.Parameter(torch.zeros(W, **f32))  # applied as 1 + w
        self.canon = CausalConv(W, cfg.canon_taps, residual=True, device=device) if cfg.canon_taps else None
        self.mixer = MIXER_TYPES[spec["type"]](W, spec["mixer"], cfg.layer_norm_eps, device=device, dtype=dtype)
        mlp = spec.get("mlp")
        self.ff = ClampedGLU(W, int(mlp["ff"]), float(mlp["limit"]), device=device, dtype=dtype) if mlp is not None else None
        self.norm2 = nn.Parameter(torch.zeros(W, **f32)) if self.ff is not None else None

    def state_shapes(self):
        return ([self.canon.state_shape()] if self.canon is not None else []) + list(self.mixer.state_shapes())


class DumalixLM(nn.Module):
    is_hybrid = True

    def __init__(self, cfg: DumalixConfig, device=None, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        kw = dict(device=device, dtype=dtype)
        W = cfg.hidden
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        self.layers = nn.ModuleList([DumalixLayer(cfg, s, **kw) for s in cfg.layer_specs])
        self.loop_in = nn.Parameter(torch.empty(W, 2 * W, **kw)) if cfg.loop else None
        self.final_norm = nn.Parameter(torch.zeros(W, device=device, dtype=torch.float32))
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W, **kw))
        self.runs = cfg.runs()
        with torch.no_grad():
            self.embed.normal_(0.0, 0.02)
            self.lm_head.normal_(0.0, 0.02)
            if self.loop_in is not None:  # near [I ; 0]: a pass starts from the stream it is given
                self.loop_in.normal_(0.0, 0.02)
                self.loop_in[:, :W] += torch.eye(W, **kw)

    @property
    def dtype(self):
        return self.embed.dtype

    @property
    def has_recurrent_state(self) -> bool:
        return any(len(l.state_shapes()) > 0 for l in self.layers)

    def head_weight(self):
        return self.lm_head

    def cache_kinds(self):
        """One cache entry per layer run: a paged pool of the mixer's rows and the run's state pools
        (input convolution first, then the mixer's)."""
        return [("rows+state", (self.layers[i].mixer.cache_row, self.layers[i].state_shapes())) for i, _ in self.runs]

    # ------------------------------------------------------------------ serving step
    def _enter_pass(self, x: torch.Tensor, x0: torch.Tensor) -> torch.Tensor:
        """x <- W_in [x ; x0]: the product's inputs in the activation dtype, its result fp32."""
        xin = torch.cat([x, x0], 1).to(self.dtype)
        if xin.dtype == torch.float32:
            return F.linear(xin, self.loop_in)
        try:
            return torch.mm(xin, self.loop_in.t(), out_dtype=torch.float32)
        except (TypeError, RuntimeError):
            return F.linear(xin, self.loop_in).float()

    def step(self, b: StepBatch, cache, rows: Optional[torch.Tensor] = None, trail: Optional[list] = None):
        """Run the step's packed tokens through all layer runs against the engine's cache
        (``cache.layer(r)``: the rows and states of run r).  Returns the fp32 residual stream of ``rows``
        (all rows if None) after the last run; ``trail`` collects it after every run."""
        eps, dt = self.cfg.layer_norm_eps, self.dtype
        x0 = F.embedding(b.ids, self.embed).float()
        x = x0.clone()
        y = z = None  # the previous run's branches, not yet added to x
        nr = len(self.runs)
        for r, (i, first) in enumerate(self.runs):
            layer = self.layers[i]
            if first:
                if y is not None:
                    hops.residual_add_act_(x, y, z)
                    y = z = None
                x = self._enter_pass(x, x0)
            h1, h2 = hops.add_rmsnorm2_f32_(x, y, z, layer.norm1, layer.norm2, eps, True, dt)
            rows_r, states = cache.layer(r)
            if layer.canon is not None:
                h1 = layer.canon(h1, b, states[0])
                states = states[1:]
            y = layer.mixer.step(h1, b, (rows_r, states))
            z = layer.ff(h2) if layer.ff is not None else None
            if trail is not None:
                hops.residual_add_act_(x, y, z)
                y = z = None
                trail.append(x.clone())
        if y is not None:
            hops.residual_add_act_(x, y, z)
        return x if rows is None else x.index_select(0, rows)

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        xn, _ = hops.add_rmsnorm2_f32_(x.contiguous(), None, None, self.final_norm, None, self.cfg.layer_norm_eps, True,
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
        put(self.final_norm, W["final.norm"])
        if self.loop_in is not None:
            put(self.loop_in, W["loop.in"])
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            put(layer.norm1, W[p + "norm1"])
            if layer.canon is not None:
                put(layer.canon.weight, W[p + "canon1"])
            m, q = layer.mixer, p + "mix."
            if isinstance(m, GroupedAttention):
                put(m.w_qkv, torch.cat([W[q + "q"], W[q + "k"], W[q + "v"]], 0))
                if m.conv is not None:
                    put(m.conv.weight, torch.cat([W[q + "q.conv"], W[q + "k.conv"], W[q + "v.conv"]], 0))
                put(m.q_norm, W[q + "q.norm"])
                put(m.k_norm, W[q + "k.norm"])
                put(m.temp, W[q + "temp"])
                put(m.sink, W[q + "sink"])
                put(m.w_o, W[q + "o"])
            else:
                put(m.w_in, torch.cat([W[q + "q"], W[q + "dkv"]], 0))
                put(m.kv_norm, W[q + "dkv.norm"])
                put(m.w_uk.view(m.H * m.dn, m.rk), W[q + "uk"])
                put(m.w_uv.view(m.H * m.dv, m.rk), W[q + "uv"])
                put(m.w_o, W[q + "o"])
            if layer.ff is not None:
                put(layer.norm2, W[p + "norm2"])
                put(layer.ff.w_gu, torch.cat([W[p + "mlp.gate"], W[p + "mlp.up"]], 0))
                put(layer.ff.w_down, W[p + "mlp.down"])

    @torch.no_grad()
    def export_named(self) -> Dict[str, torch.Tensor]:
        """The inverse of :meth:`load_named`: tensors under the checkpoint's names."""
        out = {"embed": self.embed, "head": self.lm_head, "final.norm": self.final_norm}
        if self.loop_in is not None:
            out["loop.in"] = self.loop_in
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = layer.norm1
            if layer.canon is not None:
                out[p + "canon1"] = layer.canon.weight
            m, q = layer.mixer, p + "mix."
            if isinstance(m, GroupedAttention):
                a, c = m.H * m.dk, (m.H + m.G) * m.dk
                out.update({q + "q": m.w_qkv[:a], q + "k": m.w_qkv[a:c], q + "v": m.w_qkv[c:], q + "q.norm": m.q_norm,
                            q + "k.norm": m.k_norm, q + "temp": m.temp, q + "sink": m.sink, q + "o": m.w_o})
                if m.conv is not None:
                    w = m.conv.weight
                    out.update({q + "q.conv": w[:a], q + "k.conv": w[a:c], q + "v.conv": w[c:]})
            else:
                a = m.q_cols
                out.update({q + "q": m.w_in[:a], q + "dkv": m.w_in[a:], q + "dkv.norm": m.kv_norm,
                            q + "uk": m.w_uk.reshape(m.H * m.dn, m.rk), q + "uv": m.w_uv.reshape(m.H * m.dv, m.rk),
                            q + "o": m.w_o})
            if layer.ff is not None:
                ff = layer.ff.ff
                out.update({p + "norm2": layer.norm2, p + "mlp.gate": layer.ff.w_gu[:ff], p + "mlp.up": layer.ff.w_gu[ff:],
                            p + "mlp.down": layer.ff.w_down})
        return {k: v.detach().clone().contiguous() for k, v in out.items()}


def load_dumalix(ck: Path, cfg: DumalixConfig, device=None, dtype=torch.bfloat16) -> DumalixLM:
    from safetensors import safe_open

    with safe_open(str(ck / "model.safetensors"), framework="pt", device="cpu") as f:
        W = {k: f.get_tensor(k) for k in f.keys()}
    # the convolutions' tap counts are the tensors' second size; they win over (or stand in for) the config's
    if "l0.canon1" in W:
        cfg.canon_taps = int(W["l0.canon1"].shape[1])
    for i, spec in enumerate(cfg.layer_specs):
        if spec["type"] == "attention":
            w = W.get(f"l{i}.mix.q.conv")
            spec["mixer"]["conv"] = int(w.shape[1]) if w is not None else 0
    model = DumalixLM(cfg, device=device, dtype=dtype)
    model.load_named(W)
    return model


def dumalix_template(width: int = 256, layers: int = 4, heads: int = 4, kv_heads: int = 2, vocab: int = 512, every: int = 2,
                     ff: Optional[int] = None, chunk: int = 256, taps: int = 4, loop: Optional[Tuple[int, int, int]] = None,
                     head_dim: Optional[int] = None) -> DumalixConfig:
    """A random-init configuration for benchmarks and smoke runs: latent attention in every layer but
    each ``every``-th, which is chunked grouped-query attention; sizes scale with ``width`` and ``heads``."""
    d = head_dim or width // heads
    rot = max(d // 2, 2) // 2 * 2
    yarn = {"factor": 4.0, "original": 1024, "fast": 32.0, "slow": 1.0}
    lat = {"heads": heads, "dim": d, "rot_dim": rot, "vdim": d, "kv_rank": min(max(width // 4, 8), 512),
           "rot": {"base": 10000.0, "dims": rot, "scaling": dict(yarn)}, "scale": (d + rot) ** -0.5}
    att = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "conv": taps, "mask": {"size": chunk},
           "rot": {"base": 500000.0, "dims": d // 2 * 2, "scaling": dict(yarn)}, "scale": d ** -0.5}
    mlp = {"kind": "dense", "ff": ff or 3 * width // 2, "limit": 7.0}
    specs = [{"type": "attention" if (i + 1) % every == 0 else "latent_attention",
              "mixer": copy.deepcopy(att if (i + 1) % every == 0 else lat), "mlp": copy.deepcopy(mlp)}
             for i in range(layers)]
    lp = {"start": loop[0], "stop": loop[1], "times": loop[2]} if loop else None
    return DumalixConfig(name=f"dumalix-w{width}-l{layers}", vocab_size=vocab, hidden=width, layer_specs=specs,
                         layer_norm_eps=1e-5, canon_taps=taps, loop=lp)
