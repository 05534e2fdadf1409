"""Trace replay: drive the engine's own step function with given token ids.

It samples nothing and has no forward pass, cache or loader of its own: each line of
input becomes one call of :meth:`Runner.step`, the same call generation makes.

Input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: per request its next tokens and the places among them whose logits are
wanted.  ``end``: requests that are over after this step; their pages go back to the
pool.  For a step in which something is wanted, ``<out>/<step>.f32`` receives the logits
as little-endian float32 ``[wanted, vocab]``, in the order of the entries and of
``want``.  After every step a line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Dict

PAGE_SIZE = 64  # pool pages are counted in units of 64 tokens, as --max-tokens is
MAX_LIVE = 8


def _note(text: str) -> None:
    print(f"[trace_run] {text}", file=sys.stderr, flush=True)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", required=True, type=int,
                        help="most tokens live requests hold at once (each rounded up to 64)")
    args = parser.parse_args(argv)
    if args.max_tokens < 1:
        parser.error("--max-tokens must be positive")

    _note("loading kernels (compiled at the first call) ...")
    from ..kernels import load

    load()
    import torch

    from .batch import StepEntry
    from .runner import Runner

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    num_pages = (args.max_tokens + PAGE_SIZE - 1) // PAGE_SIZE
    _note(f"loading {args.model} as {args.dtype}; cache of {num_pages} pages of {PAGE_SIZE} tokens")
    runner = Runner.from_folder(args.model, dtype=args.dtype, page_size=PAGE_SIZE,
                                num_pages=num_pages, max_requests=MAX_LIVE)
    live: Dict[str, object] = {}
    _note("ready")
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            rid = item["id"]
            if not item["tokens"]:
                continue  # nothing to run for this request in this step
            seq = live.get(rid)
            if seq is None:
                seq = live[rid] = runner.open(rid)
            entries.append(StepEntry(seq, item["tokens"], item.get("want", ())))
        if entries:
            logits = runner.step(entries)
            if logits is not None:
                data = logits.to(torch.float32).cpu().contiguous().numpy()
                data.astype("<f4", copy=False).tofile(out_dir / f"{step}.f32")
        for rid in record.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                runner.close(seq)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
