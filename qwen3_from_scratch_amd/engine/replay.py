"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it
drives the same runner (model, step function, cache manager, kernels) that
generation uses. The reference has no such tool; the nearest are
BatchRunner.prefill/step (src/qwen3_from_scratch/inference/engine.py:129-172).

Input, one JSON object per line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` receives the logits
at the wanted places as little-endian float32 [wanted, vocab], in the order of
the entries and of `want`. After every step a line `done <step>` is printed.
"""

import argparse
import json
import os
import sys


def main(argv=None):
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to 64)")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--max-requests", type=int, default=8)
    args = parser.parse_args(argv)

    import numpy as np
    import torch

    from .batch import StepEntry
    from .loading import load_runner

    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; this engine has no host implementation", file=sys.stderr)
        return 3
    os.makedirs(args.out, exist_ok=True)
    runner = load_runner(args.model, dtype=args.dtype, device="cuda", page_size=args.page_size,
                         max_tokens=args.max_tokens, max_requests=args.max_requests)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = [StepEntry(e["id"], list(e["tokens"]), list(e.get("want", [])))
                   for e in record.get("entries", [])]
        logits = runner.step(entries)
        if logits.shape[0]:
            data = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            with open(os.path.join(args.out, "%s.f32" % step), "wb") as fh:
                fh.write(np.ascontiguousarray(data).tobytes())
        else:
            torch.cuda.synchronize()
        for rid in record.get("end", []):
            runner.finish(rid)
        print("done %s" % step, flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
