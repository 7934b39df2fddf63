"""Helpers of the Lenitar tests: small configurations, random checkpoints written from the naming
rules of the checkpoint layout (not from the model class), an engine on them, and a driver that runs a
schedule of portions through ``InferenceEngine.forward_portions`` and collects every position's logits."""

from __future__ import annotations

import json
import math
from typing import Dict, List, Tuple

import torch

from llmctl.serve.engine import InferenceEngine
from llmctl.serve.scheduler import PrefillChunk


def attn(heads=2, dim=8, rot_dim=8, vdim=6, kv_rank=16, q_rank=10, window=5, base=100.0, rot_dims=None, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "rot": {"base": base, "dims": rot_dims if rot_dims is not None else rot_dim},
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "mask": {"size": window}}}


def rec(heads=2, dim=6, vdim=10, cap=15.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def moe(experts=6, top=2, groups=3, keep=2, ff=8):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top,
                                                            "groups": {"count": groups, "keep": keep}}}


def config(layers: List[Tuple[dict, dict]], width=24, vocab=50, eps=1e-5, scale=1.7) -> dict:
    return {"architecture": "Lenitar", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
            "layers": [dict(m, mlp=f) for m, f in layers]}


def random_weights(cfg: dict, seed: int = 0, forget_bias: float = 2.0) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).bfloat16().float()

    def vec(n, mean=0.0, std=1.0):
        return (mean + std * torch.randn(n, generator=g)).bfloat16().float()

    out = {"embed": vec(cfg["vocab"] * W).view(cfg["vocab"], W), "head": lin(cfg["vocab"], W),
           "final.norm": vec(W, 1.0, 0.1), "final.norm.b": vec(W, 0.0, 0.1)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"], out[p + "norm1.b"] = vec(W, 1.0, 0.1), vec(W, 0.0, 0.1)
        q = p + "mix."
        if layer["type"] == "latent_attention":
            H, dn, dr, dv, rk, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({q + "dq": lin(qr, W), q + "dq.norm": vec(qr, 1.0, 0.1), q + "uq": lin(H * (dn + dr), qr, 2.0),
                        q + "dkv": lin(rk + dr, W), q + "dkv.norm": vec(rk, 1.0, 0.1), q + "uk": lin(H * dn, rk, 2.0),
                        q + "uv": lin(H * dv, rk), q + "sink": vec(H), q + "g": lin(H * dv, W), q + "o": lin(W, H * dv)})
        else:
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            out.update({q + "q": lin(H * dk, W), q + "k": lin(H * dk, W), q + "v": lin(H * dv, W), q + "g": lin(H * dv, W),
                        q + "o": lin(W, H * dv), q + "norm": vec(H * dv, 1.0, 0.1), q + "i": lin(H, W),
                        q + "i.b": vec(H, 0.0, 0.5), q + "f": lin(H, W), q + "f.b": vec(H, forget_bias, 0.5)})
        f = layer.get("mlp")
        if f is not None:
            r, ff = f["router"], f["expert"]["ff"]
            out[p + "mlp.router"] = lin(r["experts"], W, 3.0)
            for e in range(r["experts"]):
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = lin(ff, W), lin(ff, W)
                out[f"{p}mlp.e{e}.down"] = lin(W, ff)
    return out


def write_checkpoint(path, cfg: dict, W: Dict[str, torch.Tensor]) -> str:
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()}, str(path / "model.safetensors"))
    return str(path)


def engine(path: str, device: str, dtype=torch.float32, blocks=64, block_size=4, max_seqs=4, **kw) -> InferenceEngine:
    return InferenceEngine(path, device=device, dtype=dtype, max_batch_size=max_seqs, num_kv_blocks=blocks,
                           block_size=block_size, max_model_len=blocks * block_size, max_batch_tokens=1 << 20,
                           use_graphs=False, **{"prefix_caching": False, **kw})


def run_schedule(eng: InferenceEngine, requests: Dict[str, List[int]], steps: List[List[Tuple[str, int]]]):
    """Run ``steps`` (each a list of (request, token count) that form ONE engine step); a request ends
    when its tokens are used up.  Returns request -> logits [tokens, vocab] (fp32, CPU) of every position."""
    live, at, got = {}, {k: 0 for k in requests}, {k: [] for k in requests}
    for step in steps:
        portions, want = [], []
        for rid, count in step:
            toks = requests[rid][at[rid]:at[rid] + count]
            if rid not in live:
                live[rid] = eng.open_sequence(toks, request_id=rid)
            else:
                eng.extend_sequence(live[rid], toks)
            portions.append(PrefillChunk(live[rid], live[rid].num_computed, count))
            want.append(list(range(count)))
            at[rid] += count
        logits = eng.forward_portions(portions, want).float().cpu()
        o = 0
        for rid, count in step:
            got[rid].append(logits[o:o + count])
            o += count
        for rid, _ in step:
            if at[rid] == len(requests[rid]) and rid in live:
                eng.scheduler.finish(live.pop(rid), "stop")
    return {k: torch.cat(v) for k, v in got.items() if v}


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest per-position RMS difference of the centred logits, relative to the RMS of the wanted ones."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())
