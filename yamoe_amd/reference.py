"""`yamoe.reference` of drbh/yamoe (perf_plot.py:23): the torch GPT-OSS experts module the sweep is compared with."""
from .torch_baseline import GptOssExperts

__all__ = ["GptOssExperts"]
