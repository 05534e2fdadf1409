"""The engine against the plain implementation under every way of cutting the work:
each request alone and whole; most of it in one step and the last 32 tokens one by one;
portions of changing size; and mixed batches of up to four live requests with so few
pages that they are used again.  In float32 and in bfloat16, through the step function
in-process and through the replay program as a user runs it."""
import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from tests import traces
from tests.helpers import CONFIGS, make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent

# Absolute error bounds on logits, as a fraction of the largest |logit| of the same position.
# float32: accumulated rounding of a few hundred float32 operations per output.
# bfloat16: activations are rounded to 8 bits of mantissa a few times per layer.
BOUND = {"float32": 2e-5, "bfloat16": 2e-2}
# Between two cuttings of the same work: float32 kernels give every output by one fixed
# chain of operations, so cuttings agree to the bit; bfloat16 matrix products may pick
# another library kernel for another batch size.
CUT_BOUND = {"float32": 0.0, "bfloat16": 1e-2}

LENGTHS = {"A": (5, 17, 33, 97, 128), "B": (1, 31, 64, 100, 200, 256), "C": (40, 333, 70, 129),
           "D": (2, 150, 2100, 65), "E": (3, 200, 70, 450)}


def requests_for(name):
    vocab = CONFIGS[name]["vocab_size"]
    return {f"r{i}": random_tokens(vocab, n, 50 + i) for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    tmp = tmp_path_factory.mktemp("models")
    out = {}
    for name in CONFIGS:
        for dtype in ("float32", "bfloat16"):
            folder = make_model_folder(tmp, name, dtype=dtype)
            cfg, weights = read_folder(folder)
            want = {rid: plain.forward(weights, cfg, toks) for rid, toks in requests_for(name).items()}
            out[name, dtype] = (folder, cfg, want)
    return out


def run_steps(folder, dtype, steps, *, page_size=64, max_tokens=None, vocab):
    """Drive Runner.step with the trace, the way the replay program does."""
    from pylon_amd.engine import Runner

    max_tokens = max_tokens or traces.peak_tokens(steps, page_size)
    runner = Runner.from_folder(folder, dtype=dtype, page_size=page_size,
                                num_pages=-(-max_tokens // page_size), max_requests=8)
    return traces.replay(runner, steps, vocab)


def check(got, want, dtype, what):
    for rid, ref in want.items():
        frac = np.abs(got[rid] - ref).max(axis=1) / np.abs(ref).max(axis=1)
        assert frac.max() <= BOUND[dtype], (
            f"{what}: request {rid}: first bad position {int(np.argmax(frac > BOUND[dtype]))}, "
            f"worst {int(frac.argmax())} off by {frac.max():.3e} of its largest logit")


CUTTINGS = {
    "whole": traces.whole,
    "tail32": traces.tail_one_by_one,
    "portions": traces.changing_portions,
    "mixed": lambda reqs: traces.mixed(reqs, seed=7),
    "mixed_other": lambda reqs: traces.mixed(reqs, seed=8, live_limit=3, max_portion=11),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_cutting_matches_the_plain_implementation(folders, name, dtype):
    folder, cfg, want = folders[name, dtype]
    reqs = requests_for(name)
    results = {}
    for cut, make in CUTTINGS.items():
        steps = make(reqs)
        got, reused = run_steps(folder, dtype, steps, vocab=cfg["vocab_size"])
        check(got, want, dtype, f"{name}/{dtype}/{cut}")
        results[cut] = got
        if cut.startswith("mixed"):
            assert reused, "the mixed trace was meant to use pages again"
            assert max(len(s["entries"]) for s in steps) >= 3
            assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"] if len(s["entries"]) > 1)
    for cut, got in results.items():
        for rid in want:
            ok, row, frac = rows_within(got[rid], results["whole"][rid], CUT_BOUND[dtype])
            assert ok, f"{name}/{dtype}: {cut} differs from whole at position {row} by {frac:.3e} of its scale"


@pytest.mark.parametrize("page_size", [16, 32, 256])
def test_logits_do_not_depend_on_the_page_size(folders, page_size):
    folder, cfg, want = folders["B", "float32"]
    reqs = requests_for("B")
    steps = traces.mixed(reqs, seed=11)
    got, _ = run_steps(folder, "float32", steps, page_size=page_size, vocab=cfg["vocab_size"])
    check(got, want, "float32", f"page size {page_size}")
    base, _ = run_steps(folder, "float32", steps, page_size=64, vocab=cfg["vocab_size"])
    for rid in want:
        assert np.array_equal(got[rid], base[rid])


def test_stale_pages_do_not_leak_into_later_requests(folders):
    """Pages that come back hold the old request's keys.  Poison every free page with
    NaN between steps: a kernel that reads past a request's own tokens shows at once."""
    from pylon_amd.engine import Runner, StepEntry

    folder, cfg, want = folders["A", "float32"]
    reqs = requests_for("A")
    steps = traces.mixed(reqs, seed=21)
    runner = Runner.from_folder(folder, dtype="float32", page_size=16,
                                num_pages=-(-traces.peak_tokens(steps, 16) // 16), max_requests=8)
    live, outputs = {}, {}
    group = runner.manager.groups[0]
    for step in steps:
        for page in group.pool._free:
            for c in group.cache_ids:
                group.k[c][page] = float("nan")
                group.v[c][page] = float("nan")
        entries = []
        for e in step["entries"]:
            if e["id"] not in live:
                live[e["id"]] = runner.open(e["id"])
            entries.append(StepEntry(live[e["id"]], e["tokens"], e["want"]))
        outputs[step["step"]] = runner.step(entries).cpu().numpy()
        for rid in step["end"]:
            runner.close(live.pop(rid))
    got = traces.collect(steps, outputs, cfg["vocab_size"])
    check(got, want, "float32", "poisoned free pages")


def test_a_refused_step_leaves_the_cache_as_it_was(folders):
    from pylon_amd.cache import OutOfPages
    from pylon_amd.engine import Runner, StepEntry

    folder, cfg, want = folders["A", "float32"]
    toks = requests_for("A")["r3"]
    runner = Runner.from_folder(folder, dtype="float32", page_size=16, num_pages=7, max_requests=4)
    a, b = runner.open("a"), runner.open("b")
    first = runner.step([StepEntry(a, toks[:40], list(range(40)))]).cpu().numpy()
    with pytest.raises(OutOfPages):
        runner.step([StepEntry(a, toks[40:50], []), StepEntry(b, toks[:70], [])])  # needs 1 + 5, 4 free
    assert a.length == 40 and b.length == 0 and runner.manager.free_pages == 4
    with pytest.raises(ValueError, match="Token IDs"):
        runner.step([StepEntry(a, [cfg["vocab_size"]], [0])])
    with pytest.raises(ValueError, match="at most 128 tokens"):
        runner.step([StepEntry(b, [1] * 129, [])])
    rest = runner.step([StepEntry(a, toks[40:], list(range(len(toks) - 40)))]).cpu().numpy()
    got = np.concatenate([first, rest])
    ok, row, frac = rows_within(got, want["r3"], BOUND["float32"])
    assert ok, f"position {row} is off by {frac:.3e} of its largest logit"
    runner.manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program_as_a_user_runs_it(folders, tmp_path, dtype):
    folder, cfg, want = folders["B", dtype]
    reqs = requests_for("B")
    steps = traces.mixed(reqs, seed=5)
    # one step asks for nothing: no file is written for it
    steps[0]["entries"] = [dict(e, want=[]) for e in steps[0]["entries"]]
    out = tmp_path / "out"
    proc = subprocess.Popen(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(traces.peak_tokens(steps))],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, cwd=str(tmp_path),
        env=dict(os.environ, PYTHONUNBUFFERED="1"))
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {step['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    assert not (out / "0.f32").exists()
    outputs = {}
    for step in steps[1:]:
        wanted = sum(len(e["want"]) for e in step["entries"])
        data = np.fromfile(out / f"{step['step']}.f32", dtype="<f4")
        assert data.size == wanted * cfg["vocab_size"]
        outputs[step["step"]] = data.reshape(wanted, cfg["vocab_size"])
    got = traces.collect(steps, outputs, cfg["vocab_size"])
    first = steps[0]["entries"]
    for rid, ref in want.items():
        skipped = next((len(e["tokens"]) for e in first if e["id"] == rid), 0)
        if skipped == len(ref):
            assert rid not in got  # all of it ran in the step that asked for nothing
            continue
        ok, row, frac = rows_within(got[rid], ref[skipped:], BOUND[dtype])
        assert ok, f"{rid}: position {skipped + row} is off by {frac:.3e} of its largest logit"
