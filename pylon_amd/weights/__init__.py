from .loader import WeightsError, load_weights, shard_files
from .random_init import fill_random_model, write_random_model

__all__ = ["WeightsError", "load_weights", "shard_files", "write_random_model", "fill_random_model"]
