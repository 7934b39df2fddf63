"""Replay a token trace through the serving engine and write the logits it asks for.

    python -m llmctl.serve.trace_replay --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:
``{"step": n, "entries": [{"id": "a", "tokens": [...], "want": [...]}, ...], "end": ["a", ...]}``.
Every step's entries run as ONE engine step (prompt portions beside single decoded tokens) from the
cache and state that earlier steps left; the logits at the wanted places go to ``OUT/<n>.f32``
(little-endian fp32 ``[wanted, vocab]``, entry order) and ``done <n>`` is printed after every step.
Nothing is sampled.  The engine's cache pool holds ``--max-tokens`` tokens and ``--max-seqs`` state
slots; finished requests give their blocks and slot back.

The model class is chosen by the checkpoint's ``config.json`` (``llmctl.models.registry``); the
replay holds no model code, cache or loop of its own: it calls ``InferenceEngine.open_sequence`` /
``extend_sequence`` / ``forward_portions`` and ``scheduler.finish``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="Replay a token trace through the serving engine")
    ap.add_argument("--model", required=True, help="checkpoint directory (config.json + model.safetensors)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="directory for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, default=4096, help="tokens the cache pool holds")
    ap.add_argument("--max-seqs", type=int, default=4, help="live sequences (state slots)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--device", default="auto")
    a = ap.parse_args(argv)

    import torch

    from llmctl.serve.engine import InferenceEngine
    from llmctl.serve.scheduler import PrefillChunk

    if a.device == "auto" and torch.cuda.is_available():
        # the kernels this model family needs, built on first use in a fresh checkout
        from llmctl.ops.build import ensure_group

        ensure_group("hybrid")
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    torch.backends.cuda.matmul.allow_tf32 = False
    bs = a.block_size
    blocks = (a.max_tokens + bs - 1) // bs
    eng = InferenceEngine(a.model, device=a.device, dtype=dtype, max_batch_size=a.max_seqs,
                          max_batch_tokens=1 << 30, max_model_len=max(a.max_tokens, bs), block_size=bs,
                          num_kv_blocks=blocks, use_graphs=False, prefix_caching=False)
    if eng.device.type == "cpu" and a.dtype == "bfloat16":
        print("note: CPU engine runs fp32", file=sys.stderr)
    os.makedirs(a.out, exist_ok=True)
    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        portions, want = [], []
        for e in step.get("entries", []):
            toks = [int(t) for t in e["tokens"]]
            seq = live.get(e["id"])
            if seq is None:
                seq = live[e["id"]] = eng.open_sequence(toks, request_id=str(e["id"]))
            else:
                eng.extend_sequence(seq, toks)
            portions.append(PrefillChunk(seq, seq.num_computed, len(toks)))
            want.append([int(w) for w in e.get("want", [])])
        if portions:
            logits = eng.forward_portions(portions, want)
            if logits.shape[0]:
                out = logits.float().cpu().numpy().astype("<f4")
                tmp = os.path.join(a.out, f".{step['step']}.part")
                out.tofile(tmp)
                os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
            elif eng.device.type == "cuda":
                torch.cuda.synchronize()
        for rid in step.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                eng.scheduler.finish(seq, "stop")
        print(f"done {step['step']}", flush=True)
    eng.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
