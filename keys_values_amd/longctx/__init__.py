"""Callers of the attention / cache path: a Qwen3-shaped chunked long-context prefill
(keys_values/long_context.py, keys_values/model.py) on the kernels of this package."""
from keys_values_amd.longctx.schedule import create_chunk_sizes  # noqa: F401
from keys_values_amd.longctx.model import PrefillConfig, LongContextPrefillModel, QWEN3_4B  # noqa: F401
