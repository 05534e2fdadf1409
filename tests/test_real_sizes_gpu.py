"""The layer sizes the benchmark runs (Qwen3-4B: width 2560, 32 query and 8 key/value heads of
128, feed-forward 9728, pages of 256 tokens), with two layers and a small vocabulary so that
the plain implementation stays quick: the kernels chosen at these sizes (the attention kernel
that loads pages straight into LDS, the weight-streaming products with K cut in parts, the
fused decode attention, decode graphs) against the plain model, whole and cut."""
import numpy as np
import pytest
import torch

from tests.helpers import make_model_folder, random_tokens, read_folder, rows_within
from tests.plain import qwen3 as plain

pytestmark = pytest.mark.gpu

REAL = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", hidden_act="silu", attention_bias=False,
    num_hidden_layers=2, hidden_size=2560, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
    intermediate_size=9728, vocab_size=2048, rope_theta=5000000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=8192,
)


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    folder = make_model_folder(tmp_path_factory.mktemp("real"), "real", dtype="bfloat16", config=REAL,
                               seed=3, norm_jitter=0.1)
    cfg, weights = read_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, 900 + n) for n in (300, 70, 17)]
    want = [plain.forward(weights, cfg, p) for p in prompts]
    return folder, cfg, prompts, want


@pytest.mark.parametrize("dtype,bound", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_benchmark_layer_sizes_match_the_plain_model(real, dtype, bound):
    from pylon_amd.engine import Runner, StepEntry

    folder, cfg, prompts, want = real
    runner = Runner.from_folder(folder, dtype=dtype, page_size=256, num_pages=8, max_requests=4)
    runner.enable_graphs(4)
    seqs = [runner.open(f"r{i}") for i in range(3)]
    # the first 270, 45 and 9 tokens as prompt portions of one step; then a mixed step (one
    # token of two requests beside ten tokens of the third); the rest decoded one by one, the
    # three requests side by side while they last: batches of 3, 2 and 1, from graphs
    cursor = [0, 0, 0]
    got = [[] for _ in prompts]

    def run(counts):
        live = [i for i in range(3) if counts[i]]
        entries = [StepEntry(seqs[i], prompts[i][cursor[i]: cursor[i] + counts[i]], list(range(counts[i])))
                   for i in live]
        out = runner.step(entries).cpu().numpy()
        at = 0
        for i in live:
            got[i].append(out[at: at + counts[i]])
            at += counts[i]
            cursor[i] += counts[i]

    run([270, 45, 9])
    run([1, 10, 1])
    while any(cursor[i] < len(prompts[i]) for i in range(3)):
        run([1 if cursor[i] < len(prompts[i]) else 0 for i in range(3)])
    assert runner.graphs.replays >= 20 and set(runner.graphs.captured_sizes()) == {1, 2, 3}
    for i, ref in enumerate(want):
        g = np.concatenate(got[i])
        assert len(g) == len(ref)
        assert rows_within(g, ref, bound)[0], (dtype, i, rows_within(g, ref, bound))


@pytest.mark.parametrize("dtype,bound", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_twenty_requests_decode_side_by_side(real, dtype, bound):
    """Batches of 17 to 64 rows: the out and down projections run on the streaming kernel with
    64 weight rows per workgroup, the other products in the library."""
    from pylon_amd.engine import Runner, StepEntry

    folder, cfg, _, _ = real
    _, weights = read_folder(folder)
    requests = [random_tokens(cfg["vocab_size"], 9 + i, 700 + i) for i in range(20)]
    want = [plain.forward(weights, cfg, r) for r in requests]
    runner = Runner.from_folder(folder, dtype=dtype, page_size=256, num_pages=20, max_requests=20)
    runner.enable_graphs(20)
    seqs = [runner.open(f"q{i}") for i in range(20)]
    decoded = 5
    runner.step([StepEntry(s, r[:-decoded], []) for s, r in zip(seqs, requests)])
    rows = []
    for t in range(decoded):
        entries = [StepEntry(s, [r[len(r) - decoded + t]], [0]) for s, r in zip(seqs, requests)]
        rows.append(runner.step(entries).cpu().numpy())
    assert runner.graphs.captured_sizes() == (20,) and runner.graphs.replays == decoded
    for i, ref in enumerate(want):
        got = np.stack([rows[t][i] for t in range(decoded)])
        assert rows_within(got, ref[-decoded:], bound)[0], (dtype, i, rows_within(got, ref[-decoded:], bound))


WIDE = dict(REAL, num_hidden_layers=1, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
            intermediate_size=16384, vocab_size=1024, rope_theta=1000000.0, tie_word_embeddings=False)


def test_a_layer_of_the_widest_shape(tmp_path):
    """Width 5120 with 64 query heads over 8 key/value heads, as Qwen3-32B (the feed-forward
    narrower, to keep the plain model quick, but deep enough that the down projection's K is
    cut in eight): the norm's wide rows, groups of eight heads in decode attention, and the
    eight partial sums, for a prompt portion and for 20 requests decoding side by side."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pylon_amd.engine import Runner, StepEntry

    folder = make_model_folder(tmp_path, "wide", dtype="bfloat16", config=WIDE, seed=4, norm_jitter=0.1)
    cfg, weights = read_folder(folder)
    requests = [random_tokens(cfg["vocab_size"], 6 + 3 * i, 800 + i) for i in range(20)]
    want = [plain.forward(weights, cfg, r) for r in requests]
    runner = Runner.from_folder(folder, dtype="bfloat16", page_size=256, num_pages=20, max_requests=20)
    seqs = [runner.open(f"w{i}") for i in range(20)]
    decoded = 3
    first = runner.step([StepEntry(s, r[:-decoded], list(range(len(r) - decoded)))
                         for s, r in zip(seqs, requests)]).cpu().numpy()
    rows = [runner.step([StepEntry(s, [r[len(r) - decoded + t]], [0]) for s, r in zip(seqs, requests)]).cpu().numpy()
            for t in range(decoded)]
    at = 0
    for i, ref in enumerate(want):
        n = len(requests[i]) - decoded
        got = np.concatenate([first[at: at + n], np.stack([rows[t][i] for t in range(decoded)])])
        at += n
        assert rows_within(got, ref, 3e-2)[0], (i, rows_within(got, ref, 3e-2))


def test_logits_do_not_depend_on_how_many_requests_share_a_step(real):
    """The same request decoded alone, as one of 16, of 20, of 64 and of 100 (where the rows go
    through the weight-streaming kernel as two halves, and gate/up and the head through the
    library): up to 16 rows every
    product runs on the weight-streaming kernel, beyond that the library takes part.  Either
    way the logits are float32 sums that were never rounded to bfloat16, the residual deltas
    are float32 sums, and the activation is rounded once: what differs is the order of the
    additions.  Up to 16 rows that order is the same, and the logits agree to the bit.  Beyond,
    a float32 sum that lands on the other side of a bfloat16 rounding boundary flips a few
    activations by one unit in the last place (3 of 6,144 in the q/k/v projection measured),
    and the layers that follow amplify that (a flipped query element moved the feed-forward's
    output by 1.4e-3 of its scale): the logits then agree within the bound that holds between
    any two cuttings of the same work, and the greedy tokens are the same.  A head that rounds
    to bfloat16 for more than 16 rows fails: its logits would all be bfloat16 numbers."""
    from pylon_amd.engine import Runner, StepEntry

    folder, cfg, _, _ = real
    _, weights = read_folder(folder)
    vocab = cfg["vocab_size"]
    target = random_tokens(vocab, 23, 4242)
    decoded = 6
    others = [random_tokens(vocab, 4 + i % 9, 5000 + i) for i in range(99)]
    want = plain.forward(weights, cfg, target)[-decoded:]
    rows = {}
    for batch in (1, 2, 16, 20, 64, 100):
        runner = Runner.from_folder(folder, dtype="bfloat16", page_size=256, num_pages=batch, max_requests=batch)
        runner.enable_graphs(batch)
        seqs = [runner.open(f"b{i}") for i in range(batch)]
        prompts = [target[:-decoded]] + others[: batch - 1]
        for seq, prompt in zip(seqs, prompts):  # every prompt alone: the same cache whatever the batch
            runner.step([StepEntry(seq, prompt, [])])
        got = []
        for t in range(decoded):
            entries = [StepEntry(seqs[0], [target[len(target) - decoded + t]], [0])]
            entries += [StepEntry(s, [(7 * i + t) % vocab], [0]) for i, s in enumerate(seqs[1:])]
            got.append(runner.step(entries)[0].cpu().numpy().copy())
        assert runner.graphs.replays == decoded
        rows[batch] = np.stack(got)
        assert rows_within(rows[batch], want, 3e-2)[0], (batch, rows_within(rows[batch], want, 3e-2))
        as_bf16 = torch.from_numpy(rows[batch]).to(torch.bfloat16).float().numpy()
        assert (as_bf16 != rows[batch]).mean() > 0.5, f"batch {batch}: the logits were rounded to bfloat16"
    for batch in (2, 16):
        assert np.array_equal(rows[batch], rows[1]), f"batch {batch} differs from batch 1"
    for batch in (20, 64, 100):
        ok, row, frac = rows_within(rows[batch], rows[1], 1e-2)
        assert ok, f"batch {batch} differs from batch 1 at decoded token {row} by {frac:.2e} of its largest logit"
        assert (rows[batch].argmax(axis=1) == rows[1].argmax(axis=1)).all(), batch
