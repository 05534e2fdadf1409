"""Ways of cutting the same requests into steps, in the replay program's input format:
a list of ``{"step", "entries": [{"id", "tokens", "want"}], "end"}`` records."""
from __future__ import annotations

import random
from typing import Dict, List, Sequence


def whole(requests: Dict[str, Sequence[int]]) -> List[dict]:
    """Each request alone and whole, one after the other."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(toks),
                                                       "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def tail_one_by_one(requests: Dict[str, Sequence[int]], tail: int = 32) -> List[dict]:
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(toks[:head]),
                                                           "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
    return steps


def changing_portions(requests: Dict[str, Sequence[int]], sizes=(2, 3, 5, 8, 13, 21, 34, 2, 7)) -> List[dict]:
    """Portions of changing size, down to two tokens, crossing page edges at odd offsets."""
    steps = []
    for n, (rid, toks) in enumerate(requests.items()):
        pos, k = 0, n  # every request starts elsewhere in the cycle of sizes
        while pos < len(toks):
            size = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            steps.append({"step": len(steps),
                          "entries": [{"id": rid, "tokens": list(toks[pos:pos + size]),
                                       "want": list(range(size))}],
                          "end": [rid] if pos + size == len(toks) else []})
            pos += size
    return steps


def mixed(requests: Dict[str, Sequence[int]], *, seed: int, live_limit: int = 4, tail: int = 32,
          max_portion: int = 24) -> List[dict]:
    """Up to ``live_limit`` requests at a time: portions of some beside single (decoded)
    tokens of others, requests sitting out steps, new ones starting as others end."""
    rnd = random.Random(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < live_limit and (not live or rnd.random() < 0.6):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            toks = requests[rid]
            if len(live) > 1 and rnd.random() < 0.2:
                continue  # left out of this step; goes on later
            pos = live[rid]
            left = len(toks) - pos
            if left <= tail:
                size = 1
            else:
                size = min(left - tail, rnd.randint(2, max_portion))
            want = list(range(size))
            entries.append({"id": rid, "tokens": list(toks[pos:pos + size]), "want": want})
            live[rid] = pos + size
            if live[rid] == len(toks):
                ended.append(rid)
        for rid in ended:
            del live[rid]
        if entries:
            rnd.shuffle(entries)
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def peak_tokens(steps: List[dict], unit: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``unit``."""
    held: Dict[str, int] = {}
    peak = 0
    for step in steps:
        for e in step["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // unit) * unit for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return peak


def collect(steps: List[dict], outputs: Dict[int, "object"], vocab: int):
    """``{request: [position -> logits row]}`` from per-step ``[wanted, vocab]`` arrays."""
    import numpy as np

    seen: Dict[str, int] = {}
    rows: Dict[str, Dict[int, np.ndarray]] = {}
    for step in steps:
        out = outputs.get(step["step"])
        cursor = 0
        for e in step["entries"]:
            start = seen.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[start + w] = out[cursor]
                cursor += 1
            seen[e["id"]] = start + len(e["tokens"])
        assert out is None or cursor == out.shape[0]
    return {rid: np.stack([r[i] for i in sorted(r)]) for rid, r in rows.items()}


def replay(runner, steps: List[dict], vocab: int, idle: int = 0):
    """Drive ``runner.step`` with the trace, the way the replay program does.  Returns
    ({request: logits by position}, the pages that more than one request held in turn).
    ``idle``: requests the caller keeps open beside the trace's."""
    from pylon_amd.engine import StepEntry

    live, outputs = {}, {}
    reused, handed = set(), set()
    for step in steps:
        entries = []
        for e in step["entries"]:
            if e["id"] not in live:
                live[e["id"]] = runner.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        logits = runner.step(entries)
        for e in step["entries"]:
            for page in live[e["id"]].pages[0]:
                if (e["id"], page) not in handed:
                    if any(p == page for _, p in handed):
                        reused.add(page)
                    handed.add((e["id"], page))
        if logits is not None:
            outputs[step["step"]] = logits.cpu().numpy()
        for rid in step["end"]:
            runner.close(live.pop(rid))
        runner.manager.check()
    assert len(runner.manager.live_sequences()) == idle
    return collect(steps, outputs, vocab), reused
