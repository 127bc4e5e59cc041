"""``trace_run``: feed given token ids through a model step by step and write logits; nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input carries one JSON object per line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: the next tokens of each request (a request is admitted at its first entry and may skip steps) and the
indices among them whose logits are wanted; ``end``: requests that are finished after the step, whose pages and state
slot go back to the pool.  All entries of a step are one batch of the engine.  For a step with wanted rows the float32
logits [rows, vocab] (little endian) are written to ``<out>/<step>.f32``; after every step ``done <step>`` is printed.

The model class is chosen by ``config.json``; engine, cache pool and kernels are those that generation and serving use
(``models/ragged_engine.py``, ``models/paged.py``, ``ops/ragged.py``).  ``--max-tokens`` sizes the page pool (each live
request's length rounded up to a page of 64 tokens); there are ``--slots`` state slots.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--slots", type=int, default=4)
    ap.add_argument("--device", default=None, help="default: the GPU")
    a = ap.parse_args(argv)

    import torch
    from ..models.arch import load_ragged_engine
    torch.backends.cuda.matmul.allow_tf32 = False          # float32 means float32
    device = a.device or "cuda"
    if device.startswith("cuda") and not torch.cuda.is_available():
        sys.stderr.write("trace_run: no GPU visible (pass --device cpu for the host-side statements)\n")
        return 2
    engine = load_ragged_engine(a.model, getattr(torch, a.dtype), device)
    pool = engine.ensure_pool(a.max_tokens, a.slots)
    os.makedirs(a.out, exist_ok=True)
    slot_of = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        entries, want = [], []
        for e in msg.get("entries", []):
            if e["id"] not in slot_of:
                slot_of[e["id"]] = pool.admit()
            if not e.get("tokens"):
                continue                                   # admitted, nothing to run for it in this step
            entries.append((slot_of[e["id"]], e["tokens"]))
            want.append(list(e.get("want") or []))
        if entries:
            logits = engine.step(entries, want)
            if logits.shape[0]:
                path = os.path.join(a.out, f"{msg['step']}.f32")
                logits.cpu().numpy().astype("<f4").tofile(path + ".part")
                os.replace(path + ".part", path)
        for rid in msg.get("end", []):
            if rid in slot_of:
                pool.release(slot_of.pop(rid))
        sys.stdout.write(f"done {msg['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
