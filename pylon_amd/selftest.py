"""``python main.py selftest``: a quick check of an installation on its GPU, from inside
the package.  A tiny random model is written to a temporary folder and run three ways
that must agree: a whole prompt in one step against the same tokens one by one (float32,
to the bit); bfloat16 against float32 (within the rounding of bfloat16); and greedy
generation through the engine against a loop over the step function."""
from __future__ import annotations

import tempfile

TINY = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 176, "vocab_size": 311, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 512,
}


def run(verbose: bool = True) -> None:
    import numpy as np
    import torch

    from .engine import Runner, StepEntry
    from .engine.engine import Engine
    from .sampling import Sampling
    from .weights import write_random_model

    if not torch.cuda.is_available():
        raise RuntimeError("A GPU is required.")

    def say(text: str) -> None:
        if verbose:
            print(f"selftest: {text}", flush=True)

    prompt = np.random.default_rng(3).integers(0, TINY["vocab_size"], 21).tolist()
    with tempfile.TemporaryDirectory(prefix="pylon_selftest_") as tmp:
        folder = write_random_model(tmp + "/float32", TINY, seed=1, dtype="float32", std=0.08, norm_jitter=0.1)
        exact = Runner.from_folder(folder, dtype="float32", page_size=16, num_pages=8, max_requests=2)
        whole = exact.open("whole")
        want = exact.step([StepEntry(whole, prompt, list(range(len(prompt))))]).cpu()
        single = exact.open("single")
        rows = [exact.step([StepEntry(single, [tok], [0])]).cpu()[0] for tok in prompt]
        if not torch.equal(torch.stack(rows), want):
            raise AssertionError("float32: a prompt fed whole and token by token gives different logits")
        say("float32: whole prompt == token by token, to the bit")

        greedy = []
        logits = want[-1]
        for _ in range(8):
            greedy.append(int(torch.argmax(logits)))
            logits = exact.step([StepEntry(whole, [greedy[-1]], [0])]).cpu()[0]
        exact.close(whole)
        exact.close(single)

        # the same numbers stored in bfloat16: matrices stay bfloat16 and run on the matrix-core
        # kernels (a folder stored in 32-bit would keep them in 32-bit and on the exact kernels)
        rounded = write_random_model(tmp + "/bfloat16", TINY, seed=1, dtype="bfloat16", std=0.08, norm_jitter=0.1)
        half = Runner.from_folder(rounded, dtype="bfloat16", page_size=16, num_pages=8, max_requests=2)
        if half.model.params["embed"].dtype != torch.bfloat16:
            raise AssertionError("a folder stored in bfloat16 was not loaded as bfloat16")
        seq = half.open("half")
        got = half.step([StepEntry(seq, prompt, list(range(len(prompt))))]).cpu()
        half.close(seq)
        worst = float(((got - want).abs().amax(dim=1) / want.abs().amax(dim=1)).max())
        if not worst < 3e-2:
            raise AssertionError(f"bfloat16 logits are {worst:.3f} of a row's largest logit away from float32")
        say(f"bfloat16 against float32: worst row off by {worst:.4f} of its largest logit")

        engine = Engine.from_folder(folder, dtype="float32", page_size=16, num_pages=8, max_batch_size=2)
        try:
            result, = engine.generate([prompt], Sampling(max_new_tokens=8, temperature=0.0))
        finally:
            engine.close()
        if result.output_ids != greedy:
            raise AssertionError(f"the engine generated {result.output_ids}, the step loop {greedy}")
        say(f"greedy generation through the engine: {result.output_ids}")
    say("ok")
