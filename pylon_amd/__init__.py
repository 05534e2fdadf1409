"""pylon_amd: a Qwen3-dense inference engine for one MI355X, assembled from parts."""
__version__ = "0.1.0"
