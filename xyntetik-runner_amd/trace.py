"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and has no forward pass, cache or loader of its own: it builds the
same ``ModelRunner`` that generation uses and calls its ``step``.  Steps are read
from a stream, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at the
wanted places, in the order of the entries and of ``want``, as little-endian 32-bit
floats ``[wanted, vocab]``.  After every step a line ``done <step>`` is printed.

The reference's nearest tools walk a fixed token sequence for scoring
(src/main.c:1344-1433) and teacher-force tokens in its tests
(tests/test_gpu_identity.c:91-105); decoded tokens are given, never
sampled, so an early difference cannot change later inputs
(tests/test_attn_tol.c:136).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import IO, Optional


def replay(runner, lines: IO[str], out_dir: str, report: Optional[IO[str]] = None) -> int:
    """Run every step of ``lines`` on ``runner``; returns the number of steps."""
    import numpy as np
    from .engine.batch import StepEntry
    os.makedirs(out_dir, exist_ok=True)
    report = report or sys.stdout
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                   for e in rec.get("entries", [])]
        logits = runner.step(entries)
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
            tmp = os.path.join(out_dir, f".{step}.f32.tmp")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            if runner.has(rid):
                runner.finish(rid)
        report.write(f"done {step}\n")
        report.flush()
        n += 1
    return n


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="replay token traces through the engine and dump logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to the page size)")
    ap.add_argument("--page-size", type=int, default=64, help="positions per cache page (a power of two, default 64)")
    ap.add_argument("--max-requests", type=int, default=16, help="most requests live at a time")
    args = ap.parse_args(argv)
    from .engine.runner import ModelRunner
    runner = ModelRunner.from_folder(args.model, dtype=args.dtype, max_tokens=args.max_tokens,
                                     page_size=args.page_size, max_requests=args.max_requests)
    replay(runner, sys.stdin, args.out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
