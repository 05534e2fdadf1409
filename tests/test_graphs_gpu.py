"""Decode-only steps replayed from HIP graphs give what the same steps give kernel by
kernel, over many replays with other work and synchronisations in between, while requests
join and leave (so batch sizes change) and pages are used again."""
import numpy as np
import pytest
import torch

from tests.helpers import make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,name", [("float32", "A"), ("bfloat16", "B"), ("bfloat16", "C")])
def test_graph_replay_equals_eager_steps(tmp_path, dtype, name):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner, StepEntry

    folder = make_model_folder(tmp_path, name, dtype=dtype, std=0.08)
    cfg, weights = read_folder(folder)
    vocab = cfg["vocab_size"]
    prompts = {f"g{i}": random_tokens(vocab, n, 300 + i) for i, n in enumerate((3, 20, 33, 9))}
    decode = {rid: random_tokens(vocab, 40, 400 + i) for i, rid in enumerate(prompts)}

    def run(graphs):
        runner = Runner.from_folder(folder, dtype=dtype, page_size=16, num_pages=24, max_requests=4)
        if graphs:
            runner.enable_graphs(4, max_tokens_per_request=96)
        live, rows = {}, {rid: [] for rid in prompts}
        order = list(prompts)
        for step in range(40):
            # requests join one after the other and leave at different times
            if step % 3 == 0 and order:
                rid = order.pop(0)
                live[rid] = runner.open(rid)
                out = runner.step([StepEntry(live[rid], prompts[rid], [len(prompts[rid]) - 1])])
                rows[rid].append(out[0].cpu().numpy())
            torch.cuda.synchronize()
            entries, who = [], []
            for rid, seq in live.items():
                i = seq.length - len(prompts[rid])
                entries.append(StepEntry(seq, [decode[rid][i]], [0]))
                who.append(rid)
            if entries:
                out = runner.step(entries).cpu().numpy()
                for r, rid in enumerate(who):
                    rows[rid].append(out[r])
            for rid in list(live):
                done = live[rid].length - len(prompts[rid])
                if done >= (12, 40, 25, 31)[list(prompts).index(rid)]:
                    runner.close(live.pop(rid))
            runner.manager.check()
        return runner, {rid: np.stack(r) for rid, r in rows.items()}

    eager_runner, eager = run(False)
    graph_runner, graphed = run(True)
    assert graph_runner.graphs.replays > 30 and set(graph_runner.graphs.captured_sizes()) >= {1, 2, 3}
    bound = 0.0 if dtype == "float32" else 1e-2
    for rid in prompts:
        assert eager[rid].shape == graphed[rid].shape
        assert rows_within(graphed[rid], eager[rid], bound)[0], rid
        # and both are the plain model's logits
        n = eager[rid].shape[0]
        toks = prompts[rid] + decode[rid][: n - 1]
        want = plain.forward(weights, cfg, toks)[len(prompts[rid]) - 1:]
        tol = 2e-5 if dtype == "float32" else 2e-2
        assert rows_within(graphed[rid], want, tol)[0], (rid, rows_within(graphed[rid], want, tol))


def test_a_request_longer_than_the_captured_table_runs_eagerly(tmp_path):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner, StepEntry

    folder = make_model_folder(tmp_path, "C", dtype="bfloat16", std=0.08)
    cfg, _ = read_folder(folder)
    runner = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=12, max_requests=2)
    runner.enable_graphs(2, max_tokens_per_request=32)
    seq = runner.open("x")
    toks = random_tokens(cfg["vocab_size"], 60, 1)
    runner.step([StepEntry(seq, toks[:28], [])])
    for t in toks[28:40]:
        runner.step([StepEntry(seq, [t], [0])])
    assert runner.graphs.replays == 4 and seq.length == 40  # positions 28..31 fit the table


def test_long_requests_share_their_keys_between_workgroups_in_graphs_too(tmp_path):
    """Two requests around a thousand tokens, decoded while they cross the length bound
    that a graph is recorded for: with and without graphs, the decode attention cuts their
    keys over several workgroups, and both give the plain model's logits."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner, StepEntry
    from pylon_amd.kernels import ops

    folder = make_model_folder(tmp_path, "D", dtype="bfloat16", std=0.08)
    cfg, weights = read_folder(folder)
    vocab = cfg["vocab_size"]
    prompts = {"long": random_tokens(vocab, 2030, 1), "other": random_tokens(vocab, 700, 2)}
    decode = {rid: random_tokens(vocab, 40, 10 + i) for i, rid in enumerate(prompts)}
    assert ops.decode_cuts(2, cfg["num_key_value_heads"], 2048) > 1

    def run(graphs):
        runner = Runner.from_folder(folder, dtype="bfloat16", page_size=64, num_pages=48, max_requests=2)
        if graphs:
            runner.enable_graphs(2, max_tokens_per_request=4096)
        seqs = {rid: runner.open(rid) for rid in prompts}
        rows = {rid: [] for rid in prompts}
        for rid, seq in seqs.items():
            out = runner.step([StepEntry(seq, prompts[rid], [len(prompts[rid]) - 1])])
            rows[rid].append(out[0].cpu().numpy())
        for i in range(39):
            out = runner.step([StepEntry(seqs[rid], [decode[rid][i]], [0]) for rid in prompts]).cpu().numpy()
            for r, rid in enumerate(prompts):
                rows[rid].append(out[r])
        return runner, {rid: np.stack(r) for rid, r in rows.items()}

    eager_runner, eager = run(False)
    graph_runner, graphed = run(True)
    graphs = graph_runner.graphs
    assert set(graphs.captured) == {graphs.key(2, 2048), graphs.key(2, 4096)} and len(graphs.captured) == 2
    for rid in prompts:
        toks = prompts[rid] + decode[rid][:39]
        want = plain.forward(weights, cfg, toks)[len(prompts[rid]) - 1:]
        assert rows_within(eager[rid], want, 2e-2)[0], rid
        assert rows_within(graphed[rid], want, 2e-2)[0], rid
        assert rows_within(graphed[rid], eager[rid], 1e-2)[0], rid


def test_graphs_captured_at_start_up(tmp_path):
    """Every batch size the pool has room for is captured beforehand; later decode steps
    only replay, with the logits of the same steps run kernel by kernel; the throw-away
    requests of the capture leave nothing behind."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner, StepEntry

    folder = make_model_folder(tmp_path, "D", dtype="bfloat16", std=0.08)
    cfg, _ = read_folder(folder)
    runner = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=40, max_requests=6)
    runner.enable_graphs(6)
    assert runner.capture_graphs() == (1, 2, 3, 4, 5, 6)
    runner.manager.check()
    assert runner.manager.free_pages == 40 and not runner.manager.live_sequences()
    captured = len(runner.graphs.captured)
    eager = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=40, max_requests=6)
    prompts = [random_tokens(cfg["vocab_size"], n, 70 + n) for n in (5, 18, 31)]
    outs = []
    for r in (runner, eager):
        seqs = [r.open(f"s{i}") for i in range(3)]
        r.step([StepEntry(s, p, []) for s, p in zip(seqs, prompts)])
        rows = [r.step([StepEntry(s, [7 + t], [0]) for s in seqs[: 3 - t % 2]]).cpu().numpy() for t in range(6)]
        outs.append(np.concatenate(rows))
    assert len(runner.graphs.captured) == captured and runner.graphs.replays >= 6 + 6
    assert rows_within(outs[0], outs[1], 1e-2)[0]
    # a pool too small for the largest sizes: those are left to their first use
    small = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=3, max_requests=6)
    small.enable_graphs(6)
    assert small.capture_graphs() == (1, 2, 3)
    small.manager.check()
    assert small.manager.free_pages == 3
    # up to a given length only the graphs of the bounds that hold it are captured; by default
    # those of every bound are, by short requests, and a long request then only replays
    big = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=140, max_requests=3)
    big.enable_graphs(2)
    assert big.graphs.bounds() == (512, 1024, 2048, 4096)
    big.capture_graphs(max_tokens=1000)
    assert set(big.graphs.captured) == {big.graphs.key(rows, bound) for rows in (1, 2) for bound in (512, 1024)}
    big.capture_graphs()
    assert set(big.graphs.captured) == {big.graphs.key(rows, bound) for rows in (1, 2)
                                        for bound in (512, 1024, 2048, 4096)}
    assert len(big.graphs.captured) == 8  # two key/value heads: every bound cuts the keys otherwise
    plain_runner = Runner.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=140, max_requests=3)
    long_prompt = random_tokens(cfg["vocab_size"], 1100, 5)
    outs = []
    for r in (big, plain_runner):
        seq = r.open("long")
        r.step([StepEntry(seq, long_prompt, [])])
        outs.append(np.concatenate([r.step([StepEntry(seq, [11 + t], [0])]).cpu().numpy() for t in range(4)]))
    assert len(big.graphs.captured) == 8 and big.graphs.replays >= 8 + 4
    assert rows_within(outs[0], outs[1], 1e-2)[0]
