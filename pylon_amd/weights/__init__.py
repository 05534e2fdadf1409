from .loader import WeightsError, load_weights, shard_files
from .random_init import write_random_model

__all__ = ["WeightsError", "load_weights", "shard_files", "write_random_model"]
