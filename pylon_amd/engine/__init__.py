from .batch import PENDING, MetadataArena, StepContext, StepEntry, build_step
from .model import Model

__all__ = ["PENDING", "MetadataArena", "StepContext", "StepEntry", "build_step", "Model"]
from .runner import Runner, resolve_dtype  # noqa: E402

__all__ += ["Runner", "resolve_dtype"]
