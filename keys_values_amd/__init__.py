"""
keys_values_amd: MI355X-native (gfx950) attention-with-score-sums and KV-cache kernels behind the
operator surface of awslabs/keys_values.

The compute lives in ``libkvx.so`` (hand-written HIP, C ABI in ``include/kvx.h``); this package is
the thin host side that mirrors the reference's Python operators:

* ``keys_values_amd.attention.ops``   <-> ``keys_values/attention/flashinfer_ops.py``
* ``keys_values_amd.attention.sdpa``  <-> ``keys_values/attention/flashinfer_wrapper.py`` (``FlashInferSDPA``)
* ``keys_values_amd.kvcache.quantize`` <-> ``keys_values/kvcache/quantize/pytorch.py`` (``TorchBasicQuantizer``, 8 bit)
* ``keys_values_amd.kvcache.h2o``     <-> ``keys_values/kvcache/h2o.py`` + ``attn_weights.py`` (``H2OKVCache``)

There is no CPU fallback: without the built library or without a gfx950 device the operators raise.
"""

__version__ = "0.1.0"
