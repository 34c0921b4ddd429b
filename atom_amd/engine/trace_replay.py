"""Trace replay: feeds given token ids through a model step by step and writes the
logits.  It samples nothing and has nothing of its own: the model, loader, cache and
step function are the ones generation uses (``EngineCore``).

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` receives the logits at the
wanted places, in the order of the entries and of ``want``, as little-endian float32
``[wanted, vocab]``.  After every step a line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import os
import sys

DEFAULT_PAGE_SIZE = 16    # the reference's --block-size default (atom/model_engine/arg_utils.py)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="the most tokens live requests hold at any time (each rounded up to 64)")
    parser.add_argument("--block-size", type=int, default=DEFAULT_PAGE_SIZE,
                        help="tokens a cache page holds")
    parser.add_argument("--max-requests", type=int, default=8, help="state slots (live requests at a time)")
    parser.add_argument("--enforce-eager", action="store_true", help="never replay captured HIP graphs")
    args = parser.parse_args(argv)
    page_size = args.block_size
    if page_size <= 0:
        parser.error("--block-size must be positive")

    def say(msg):
        print(f"[trace_run] {msg}", file=sys.stderr, flush=True)

    say("importing torch")
    import numpy as np
    import torch

    from ..kernels.hip import HipKernels
    from .core import TORCH_DTYPES, StepEntry, build_core, load_model

    dtype = TORCH_DTYPES[args.dtype]
    device = "cuda:0"
    ops = HipKernels(device)   # builds the kernel library on first use
    say(f"kernel library {ops.path}")
    model, _ = load_model(args.model, dtype=dtype, device=device, progress=say)
    num_pages = max(1, -(-args.max_tokens // page_size))
    core = build_core(model, ops, dtype=dtype, device=device, page_size=page_size, num_pages=num_pages,
                      max_num_seqs=args.max_requests,
                      graph_sizes=None if args.enforce_eager else [1, 2, 4, 8])
    os.makedirs(args.out, exist_ok=True)
    say(f"ready: {num_pages} pages of {page_size} tokens per group, {args.dtype}")

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in record.get("entries", [])]
        logits = core.step(entries) if entries else None
        if logits is not None:
            host = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            path = os.path.join(args.out, f"{step}.f32")
            tmp = path + ".tmp"
            with open(tmp, "wb") as f:
                f.write(np.ascontiguousarray(host).tobytes())
            os.replace(tmp, path)
        else:
            torch.cuda.synchronize()
        for req in record.get("end", []):
            core.close(req)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
