from .h2o import (H2OKVCache, KVCacheParams, QuantizedH2OKVCache, QuantizedVLengthH2OKVCache,  # noqa: F401
                  VLengthH2OKVCache, create_kv_cache)
from .quantize import RowQuantizer, RowQuantizer8  # noqa: F401
from .buffers import (BlockQuantizedKeysAndValues, DefaultKeysAndValues, HipKVCacheBuffers, KeysAndValues, KVCacheBuffers, KVCacheBuffersParams,  # noqa: F401
                      QuantizedKeysAndValues, create_kv_cache_buffers)
