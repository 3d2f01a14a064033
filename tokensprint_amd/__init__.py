"""tokensprint_amd: a small, whole Qwen3 inference engine for one AMD MI355X."""

__version__ = "0.1.0"
