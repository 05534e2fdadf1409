"""pylon_amd: a Qwen3-dense inference engine for one MI355X, assembled from parts.

The programming entry point works on token ids, as the reference's does
(/root/reference/src/pylon/engine.py:241-253)::

    from pylon_amd import Engine, Sampling
    engine = Engine.from_folder("model_dir", dtype="bfloat16")   # or Engine.from_random(config_dict, seed)
    future = engine.enqueue([1, 2, 3], eos_token_id=None, sampling=Sampling(max_new_tokens=16))
    engine.run_until_idle()
    print(future.result().output_ids)

Names are imported on first use, so that importing the package neither needs a GPU nor
compiles anything.
"""
__version__ = "0.1.0"

_LAZY = {
    "Engine": ("pylon_amd.engine.engine", "Engine"),
    "GenerationResult": ("pylon_amd.engine.engine", "GenerationResult"),
    "Runner": ("pylon_amd.engine.runner", "Runner"),
    "StepEntry": ("pylon_amd.engine.batch", "StepEntry"),
    "Sampling": ("pylon_amd.sampling.params", "Sampling"),
    "PylonConfig": ("pylon_amd.config.engine_config", "PylonConfig"),
    "get_config": ("pylon_amd.config.engine_config", "get_config"),
    "write_random_model": ("pylon_amd.weights.random_init", "write_random_model"),
}


def __getattr__(name):
    try:
        module, attr = _LAZY[name]
    except KeyError:
        raise AttributeError(f"module 'pylon_amd' has no attribute {name!r}") from None
    import importlib

    return getattr(importlib.import_module(module), attr)


__all__ = list(_LAZY)
