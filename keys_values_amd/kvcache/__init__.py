from .h2o import (H2OKVCache, KVCacheParams, QuantizedH2OKVCache, QuantizedVLengthH2OKVCache,  # noqa: F401
                  VLengthH2OKVCache, create_kv_cache)
from .quantize import RowQuantizer, RowQuantizer8  # noqa: F401
