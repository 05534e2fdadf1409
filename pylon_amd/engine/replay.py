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

PAGE_SIZE = 64  # default page: pool pages are counted in units of 64 tokens, as --max-tokens is
MAX_LIVE = 8  # default number of state slots (requests live at a time)


def _note(text: str) -> None:
    print(f"[trace_run] {text}", file=sys.stderr, flush=True)


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", required=True, type=int,
                        help="most tokens live requests hold at once (each rounded up to 64)")
    parser.add_argument("--page-size", type=int, default=PAGE_SIZE,
                        help=f"tokens per cache page, a multiple of 16 (default {PAGE_SIZE})")
    parser.add_argument("--max-live", type=int, default=MAX_LIVE,
                        help=f"most requests live at a time (default {MAX_LIVE})")
    args = parser.parse_args(argv)
    if args.max_tokens < 1:
        parser.error("--max-tokens must be positive")
    if args.page_size < 16 or args.page_size % 16:
        parser.error("--page-size must be a positive multiple of 16")
    if args.max_live < 1:
        parser.error("--max-live must be positive")

    _note("loading kernels (compiled at the first call) ...")
    from ..kernels import load

    load()
    import torch

    from ..cache import OutOfPages, OutOfSlots
    from .batch import StepEntry
    from .runner import Runner

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    page_size = args.page_size
    num_pages = (args.max_tokens + page_size - 1) // page_size
    _note(f"loading {args.model} as {args.dtype}; cache of {num_pages} pages of {page_size} tokens, "
          f"{args.max_live} requests live at a time")
    runner = Runner.from_folder(args.model, dtype=args.dtype, page_size=page_size,
                                num_pages=num_pages, max_requests=args.max_live)
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
                try:
                    seq = live[rid] = runner.open(rid)
                except OutOfSlots:
                    print(f"trace_run: step {step}: request {rid!r} would be live request number "
                          f"{len(live) + 1}, but --max-live is {args.max_live}", file=sys.stderr, flush=True)
                    return 3
            entries.append(StepEntry(seq, item["tokens"], item.get("want", ())))
        if entries:
            try:
                logits = runner.step(entries)
            except OutOfPages as error:
                held = sum(-(-s.length // page_size) * page_size for s in live.values())
                print(f"trace_run: step {step}: the cache of {num_pages * page_size} tokens (--max-tokens "
                      f"{args.max_tokens}, pages of {page_size}) is full: live requests hold {held} tokens "
                      f"and this step brings {sum(len(e.tokens) for e in entries)} more ({error})",
                      file=sys.stderr, flush=True)
                return 3
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
