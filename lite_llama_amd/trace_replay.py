"""Replay of a step trace: feed given token ids through a model, step by step, and write the logits of the asked places.
Nothing is sampled.  The replay drives :class:`RaggedRunner` -- the step function, cache and kernels of the generation
engine (engine.py) -- and has no forward pass, cache or loader of its own.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object a line,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: per request its next tokens and the places among them whose logits are wanted; ``end``: requests that are
finished after this step (their blocks and slot are given back).  All entries of a step run as one batch.  For a step that
wants something, ``DIR/<step>.f32`` receives the logits ``[wanted, vocab]`` as little-endian float32, in entry order; after
every step a line ``done <step>`` goes to standard output.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (per request rounded up to the page size)")
    ap.add_argument("--max-requests", type=int, default=4, help="state slots (live requests)")
    ap.add_argument("--page-size", type=int, default=64)
    args = ap.parse_args(argv)

    from . import _lib
    from .weights import MODEL_FAMILIES, model_family

    with open(os.path.join(args.model, "config.json")) as f:
        config = json.load(f)
    if model_family(config) not in MODEL_FAMILIES:
        print(f"trace_run: the {model_family(config)!r} family has no ragged step function", file=sys.stderr)
        return 2
    _lib.use_part("ragged")  # a fresh checkout compiles the sources of this family only
    _lib.lib()

    import numpy as np
    import torch

    from .executor.ragged import RaggedRunner
    from .weights import load_pretrained

    if not torch.cuda.is_available():
        print("trace_run: no GPU (there is no CPU path)", file=sys.stderr)
        return 2
    torch.backends.cuda.matmul.allow_tf32 = False
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    model = load_pretrained(args.model, device="cuda", dtype=dtype)
    runner = RaggedRunner(model, args.max_tokens, args.max_requests, args.page_size, device="cuda")
    os.makedirs(args.out, exist_ok=True)
    slots: dict[str, int] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        entries, rows, base = [], [], 0
        for e in msg["entries"]:
            if e["id"] not in slots:
                slots[e["id"]] = runner.admit()
            if not e["tokens"]:
                continue  # (admitted, brings nothing in this step)
            entries.append((slots[e["id"]], e["tokens"]))
            rows += [base + int(w) for w in e.get("want", [])]
            base += len(e["tokens"])
        if entries:
            logits = runner.step(entries, rows)
            if rows:
                data = logits.float().cpu().numpy().astype("<f4")
                tmp = os.path.join(args.out, f".{msg['step']}.part")
                data.tofile(tmp)
                os.replace(tmp, os.path.join(args.out, f"{msg['step']}.f32"))
            runner.check_errors()
        ended = [slots.pop(i) for i in msg.get("end", []) if i in slots]
        runner.release(ended)
        sys.stdout.write(f"done {msg['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
