"""Trace replay: feeds given token ids through a model step by step and writes logits.

It samples nothing and has no forward pass, cache or loader of its own: it drives the
same model, step function, cache manager and kernels that generation uses.  The
reference has no model-level replay; its per-kernel probes write named float32 tensors
for a Python comparator (/root/reference/tests/probes/attention_misc_precision_probe.rs:
10-24), which is the manner followed here at the level of the whole model.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the
wanted places as little-endian float32 [wanted, vocab]; after every step a line
`done <step>` is printed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32", "bf16", "f32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at a time, each rounded up to a page")
    ap.add_argument("--page-size", type=int, default=64, help="tokens per cache page")
    ap.add_argument("--max-requests", type=int, default=8, help="most live requests at a time")
    args = ap.parse_args(argv)

    print("trace_run: loading (kernels are compiled on the first call)", file=sys.stderr, flush=True)
    import torch
    from .loading import load_model
    from .runner import ModelRunner, StepEntry

    os.makedirs(args.out, exist_ok=True)
    model = load_model(args.model, args.dtype, "cuda:0")
    page = args.page_size
    num_pages = max(1, -(-args.max_tokens // page))
    runner = ModelRunner(model, page_size=page, num_pages=num_pages, max_requests=args.max_requests)
    ids: Dict[str, int] = {}
    next_id = 0
    print("trace_run: ready", file=sys.stderr, flush=True)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        step = msg["step"]
        entries = []
        for e in msg.get("entries", []):
            key = str(e["id"])
            if key not in ids:
                ids[key] = next_id
                next_id += 1
                runner.add_request(ids[key])
            entries.append(StepEntry(ids[key], e["tokens"], e.get("want", [])))
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(args.out, f".{step}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        else:
            torch.cuda.synchronize()
        for key in msg.get("end", []):
            key = str(key)
            if key in ids:
                runner.release(ids.pop(key))
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
