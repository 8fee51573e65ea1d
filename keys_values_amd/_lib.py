"""ctypes binding of libkvx.so (the C ABI declared in include/kvx.h). No fallback of any kind."""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkvx.so")

KVX_OK, KVX_ERR_INVALID, KVX_ERR_UNSUPPORTED, KVX_ERR_HIP, KVX_ERR_WORKSPACE = 0, 1, 2, 3, 4
KVX_KV_BF16, KVX_KV_U8, KVX_KV_U4, KVX_KV_F16, KVX_KV_U8_F16, KVX_KV_U4_F16 = 0, 1, 2, 3, 4, 5


def quant_kv_dtype(num_bits: int, dtype) -> int:
    """enum kvx_kv_dtype of a quantised store of ``num_bits`` codes whose rows were (and dequantise to) ``dtype``."""
    f16 = dtype == torch.float16
    if num_bits == 4:
        return KVX_KV_U4_F16 if f16 else KVX_KV_U4
    return KVX_KV_U8_F16 if f16 else KVX_KV_U8


def elem_kv_dtype(dtype) -> int:
    return KVX_KV_F16 if dtype == torch.float16 else KVX_KV_BF16


class SdpaArgs(ctypes.Structure):
    """struct kvx_sdpa_args"""

    _fields_ = [
        ("B", c_int32), ("Hq", c_int32), ("Hkv", c_int32), ("q_len", c_int32), ("kv_len", c_int32), ("D", c_int32),
        ("input_pos", c_int32), ("kv_dtype", c_int32), ("sm_scale", c_float), ("num_splits", c_int32),
        ("q", c_void_p), ("q_stride_b", c_int64), ("q_stride_h", c_int64), ("q_stride_t", c_int64),
        ("k", c_void_p), ("k_stride_b", c_int64), ("k_stride_h", c_int64), ("k_stride_t", c_int64),
        ("v", c_void_p), ("v_stride_b", c_int64), ("v_stride_h", c_int64), ("v_stride_t", c_int64),
        ("k_scale", c_void_p), ("k_zp", c_void_p), ("v_scale", c_void_p), ("v_zp", c_void_p),
        ("qs_stride_b", c_int64), ("qs_stride_h", c_int64),
        ("token_positions", c_void_p), ("tp_stride_b", c_int64), ("tp_stride_h", c_int64),
        ("o", c_void_p), ("o_stride_b", c_int64), ("o_stride_h", c_int64), ("o_stride_t", c_int64),
        ("lse", c_void_p), ("w", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("decode_scratch_splits", c_void_p),
    ]


class CacheWriteArgs(ctypes.Structure):
    """struct kvx_cache_write_args"""

    _fields_ = [
        ("B", c_int32), ("Hkv", c_int32), ("num", c_int32), ("D", c_int32), ("cache_len", c_int32),
        ("input_pos", c_int32), ("kv_dtype", c_int32),
        ("index", c_void_p), ("index_stride_b", c_int64), ("index_stride_h", c_int64),
        ("key", c_void_p), ("key_stride_b", c_int64), ("key_stride_h", c_int64), ("key_stride_t", c_int64),
        ("value", c_void_p), ("value_stride_b", c_int64), ("value_stride_h", c_int64), ("value_stride_t", c_int64),
        ("k_cache", c_void_p), ("kc_stride_b", c_int64), ("kc_stride_h", c_int64), ("kc_stride_t", c_int64),
        ("v_cache", c_void_p), ("vc_stride_b", c_int64), ("vc_stride_h", c_int64), ("vc_stride_t", c_int64),
        ("k_scale", c_void_p), ("k_zp", c_void_p), ("v_scale", c_void_p), ("v_zp", c_void_p),
        ("qs_stride_b", c_int64), ("qs_stride_h", c_int64),
        ("token_pos", c_void_p), ("tp_stride_b", c_int64), ("tp_stride_h", c_int64),
        ("scores", c_void_p), ("sc_stride_b", c_int64), ("sc_stride_h", c_int64),
        ("grace_num", c_int32), ("grace_period", c_int32), ("grace_slots", c_void_p),
        ("v_norm", c_void_p), ("q_errors", c_void_p),
        ("replay_log", c_void_p), ("log_blocksize", c_int32), ("log_pos", c_int64),
        ("log_stride_block", c_int64), ("log_stride_b", c_int64), ("log_stride_h", c_int64),
    ]


class H2OArgs(ctypes.Structure):
    """struct kvx_h2o_args"""

    _fields_ = [
        ("B", c_int32), ("Hkv", c_int32), ("kv_len", c_int32), ("limit", c_int32), ("k", c_int32),
        ("normalize", c_int32), ("input_pos", c_int32), ("prefill_len", c_int32),
        ("scores", c_void_p), ("sc_stride_b", c_int64), ("sc_stride_h", c_int64),
        ("w", c_void_p),
        ("token_pos", c_void_p), ("tp_stride_b", c_int64), ("tp_stride_h", c_int64),
        ("next_index", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("v_norm", c_void_p), ("q_errors", c_void_p), ("q_len", c_int32), ("combination", ctypes.c_double),
    ]


class BlockQuantArgs(ctypes.Structure):
    """struct kvx_block_quant_args"""

    _fields_ = [
        ("x", c_void_p), ("x_stride_outer", c_int64), ("x_stride_inner", c_int64), ("x_stride_seg", c_int64),
        ("n_outer", c_int32), ("n_inner", c_int32), ("nseg", c_int32), ("D", c_int32), ("bits", c_int32),
        ("codes", c_void_p), ("codes_stride_outer", c_int64),
        ("scale", c_void_p), ("zp", c_void_p), ("state_stride_outer", c_int64),
        ("elem_dtype", c_int32),
    ]


# every symbol include/kvx.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "kvx_version": (ctypes.c_int, []),
    "kvx_last_error": (c_char_p, []),
    "kvx_device_count": (ctypes.c_int, []),
    "kvx_device_info": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, c_size_t]),
    "kvx_sdpa_prefill": (ctypes.c_int, [POINTER(SdpaArgs), c_void_p]),
    "kvx_sdpa_prefill_workspace_bytes": (c_size_t, [POINTER(SdpaArgs)]),
    "kvx_score_sum": (ctypes.c_int, [POINTER(SdpaArgs), c_void_p]),
    "kvx_sdpa_prefill_weights": (ctypes.c_int, [POINTER(SdpaArgs), c_void_p]),
    "kvx_sdpa_decode": (ctypes.c_int, [POINTER(SdpaArgs), c_void_p]),
    "kvx_sdpa_decode_workspace_bytes": (c_size_t, [POINTER(SdpaArgs)]),
    "kvx_sdpa_decode_h2o": (ctypes.c_int, [POINTER(SdpaArgs), POINTER(H2OArgs), c_void_p]),
    "kvx_sdpa_decode_h2o_workspace_bytes": (c_size_t, [POINTER(SdpaArgs)]),
    "kvx_decode_tuning": (None, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "kvx_quantize_rows": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "kvx_dequantize_rows": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_int64, c_void_p]),
    "kvx_quantize_rows4": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "kvx_dequantize_rows4": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_int64, c_void_p]),
    "kvx_quantize_rows_typed": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "kvx_dequantize_rows_typed": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_void_p, c_int64, c_void_p]),
    "kvx_quantize_blocks": (ctypes.c_int, [POINTER(BlockQuantArgs), c_void_p]),
    "kvx_dequantize_blocks": (ctypes.c_int, [POINTER(BlockQuantArgs), c_void_p]),
    "kvx_cache_write": (ctypes.c_int, [POINTER(CacheWriteArgs), c_void_p]),
    "kvx_h2o_update_select": (ctypes.c_int, [POINTER(H2OArgs), c_void_p]),
    "kvx_h2o_workspace_bytes": (c_size_t, [POINTER(H2OArgs)]),
    "kvx_h2o_update_select_static": (ctypes.c_int, [POINTER(H2OArgs), c_void_p]),
    "kvx_rmsnorm_rows": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int32, ctypes.c_float, c_void_p]),
    "kvx_add_rmsnorm_rows": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                            c_int32, ctypes.c_float, c_void_p]),
    "kvx_swiglu_rows": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int32, c_void_p]),
    "kvx_qk_norm_rope": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p,
                                        ctypes.c_float, c_void_p, c_void_p, c_int32, c_int32, c_void_p]),
}

_lib = None
_load_error = None


def load():
    """Load libkvx.so and bind every symbol. Raises ImportError if the library was not built."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        _load_error = f"{LIB_PATH} not found: build it with `python -m keys_values_amd.build`"
        raise ImportError(_load_error)
    try:
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
            fn.restype = res
            fn.argtypes = args
    except (OSError, AttributeError) as ex:
        _load_error = f"{LIB_PATH}: {ex}"
        raise
    _load_error = None
    _lib = lib
    return lib


def load_error():
    return _load_error


class KvxError(RuntimeError):
    pass


def check(rc: int):
    """Translate a kvx status into the exception the reference raises in the same situation:
    shape/argument problems -> ValueError (keys_values/attention/flashinfer_wrapper.py:406-423),
    unsupported head size / dtype -> NotImplementedError (:425-432), runtime failures -> RuntimeError
    (TORCH_CHECK in keys_values/csrc/bindings.cpp:486,955)."""
    if rc == KVX_OK:
        return
    msg = load().kvx_last_error().decode("utf-8", "replace")
    if rc == KVX_ERR_INVALID:
        raise ValueError(msg)
    if rc == KVX_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise KvxError(f"kvx status {rc}: {msg}")


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t):
    return None if t is None else t.data_ptr()


def require_gpu(*tensors):
    """The kernels only run on a gfx950 device: refuse anything else loudly (no CPU path)."""
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                f"keys_values_amd: tensor on {t.device}; the HIP kernels need a ROCm device and there is no CPU fallback"
            )


_workspaces = {}


def workspace(device, nbytes: int):
    """Grow-only scratch buffer per (device, stream). Kernel launches on one stream are ordered, so
    consecutive calls may share it."""
    if nbytes == 0:
        return None
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf
