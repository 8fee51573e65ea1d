"""
Host side of the attention kernels, mirroring ``keys_values/attention/flashinfer_ops.py`` (the thin
Python layer over the reference's extension module, keys_values/csrc/bindings.cpp:1722-1844):
``is_available``, ``get_device_count``, ``get_device_info``, ``sdpa_decode``, ``sdpa_prefill``,
``sdpa_prefill_fused`` and ``sdpa_prefill_fused_v2`` keep their names, argument meaning, tensor
layouts (``[batch, len, heads, head_dim]``) and return values.

Two things differ on purpose. The functions also take the keyword arguments ``token_positions`` and
``input_pos`` (the reference's extension has them, its Python layer never passes them), so callers
need not sort the cache by position first. And the ``*_core`` functions accept any strided
``(batch, heads, len, head_dim)`` view, so the cache's own layout is read in place instead of being
transposed and copied (keys_values/attention/flashinfer_wrapper.py:590-592,667-669).

There is no fallback: a missing library or a non-ROCm tensor raises.
"""
import ctypes
import math
from typing import NamedTuple, Optional, Tuple

import torch

from .. import _lib

ALLOWED_HEAD_SIZES = (64, 128, 256)  # keys_values/attention/flashinfer_wrapper.py:276
QUANTIZED_HEAD_SIZES = ALLOWED_HEAD_SIZES  # the kernels that read codes take the same sizes
ALLOWED_DTYPES = (torch.bfloat16, torch.float16)  # keys_values/attention/flashinfer_wrapper.py:311-319


class QuantState(NamedTuple):
    """Per-row state of a quantised cache (uint8 codes of D bytes per row, or the 4-bit store of D/2 bytes per row): fp32 scales and int32 zero points, each (B, Hkv, T) with a
    contiguous last axis; K and V arrays share their strides
    (keys_values/kvcache/quantize/pytorch.py:281-295)."""

    k_scale: torch.Tensor
    k_zp: torch.Tensor
    v_scale: torch.Tensor
    v_zp: torch.Tensor


# ---- availability (keys_values/attention/flashinfer_ops.py:38-111) -------------------------------


def is_available() -> bool:
    """True iff the library loads and a gfx950 device is visible."""
    try:
        return _lib.load().kvx_device_count() > 0
    except (ImportError, OSError, AttributeError):
        return False


def get_load_error() -> Optional[str]:
    """Message of the last failed attempt to load the library, None if it loaded or was not tried
    (keys_values/attention/flashinfer_ops.py:134-147)."""
    return _lib.load_error()


def get_device_count() -> int:
    return _lib.load().kvx_device_count()


def get_device_info(device_id: int = 0) -> str:
    buf = ctypes.create_string_buffer(256)
    _lib.check(_lib.load().kvx_device_info(device_id, buf, 256))
    return buf.value.decode()


# ---- argument plumbing ----------------------------------------------------------------------------


def _check_bhtd(name: str, t: torch.Tensor):
    if t.ndim != 4:
        raise ValueError(f"{name} must be a 4D tensor, got shape {tuple(t.shape)}")
    if t.stride(-1) != 1:
        raise ValueError(f"{name}: the head dimension must be contiguous (stride {t.stride(-1)})")


def _fill_common(a: _lib.SdpaArgs, query, key, value, scale, input_pos, token_positions, quant, num_splits):
    B, Hq, q_len, D = query.shape
    _, Hkv, T, _ = key.shape
    a.B, a.Hq, a.Hkv, a.q_len, a.kv_len, a.D = B, Hq, Hkv, q_len, T, D
    a.input_pos = int(input_pos)
    a.sm_scale = float(scale)
    a.num_splits = int(num_splits)
    a.q = query.data_ptr()
    a.q_stride_b, a.q_stride_h, a.q_stride_t = query.stride(0), query.stride(1), query.stride(2)
    a.k = key.data_ptr()
    a.k_stride_b, a.k_stride_h, a.k_stride_t = key.stride(0), key.stride(1), key.stride(2)
    if value is not None:
        a.v = value.data_ptr()
        a.v_stride_b, a.v_stride_h, a.v_stride_t = value.stride(0), value.stride(1), value.stride(2)
    if quant is not None:
        # rows of D bytes: 8-bit codes; rows of D/2 bytes: the 4-bit store, two codes per byte
        a.kv_dtype = _lib.quant_kv_dtype(4 if key.shape[3] * 2 == D else 8, query.dtype)  # the rows dequantise to the query's type
        for t in quant:
            if t.shape != (B, Hkv, T) or t.stride(-1) != 1 or t.stride() != quant.k_scale.stride():
                raise ValueError("quantisation state must be (B, Hkv, T) arrays sharing strides, last axis contiguous")
        if quant.k_scale.dtype != torch.float32 or quant.k_zp.dtype != torch.int32:
            raise ValueError("quantisation state must be float32 scales and int32 zero points")
        a.k_scale, a.k_zp = quant.k_scale.data_ptr(), quant.k_zp.data_ptr()
        a.v_scale, a.v_zp = quant.v_scale.data_ptr(), quant.v_zp.data_ptr()
        a.qs_stride_b, a.qs_stride_h = quant.k_scale.stride(0), quant.k_scale.stride(1)
    else:
        a.kv_dtype = _lib.KVX_KV_F16 if query.dtype == torch.float16 else _lib.KVX_KV_BF16
    if token_positions is not None:
        a.token_positions = token_positions.data_ptr()
        a.tp_stride_b, a.tp_stride_h = token_positions.stride(0), token_positions.stride(1)


def _row_len(D: int, key: torch.Tensor, quant) -> int:
    """Last-axis length a cache row must have: D, or D/2 bytes for the 4-bit store."""
    return D // 2 if (quant is not None and key.shape[3] * 2 == D) else D


def _check_dtypes(query, key, value, quant):
    if query.dtype not in ALLOWED_DTYPES:
        raise NotImplementedError(f"query.dtype must be torch.bfloat16 or torch.float16, got {query.dtype}")
    want = torch.uint8 if quant is not None else query.dtype
    for name, t in (("key", key), ("value", value)):
        if t is not None and t.dtype != want:
            raise NotImplementedError(f"{name}.dtype must be {want}, got {t.dtype}")


def _token_positions_i32(token_positions, B, Hkv, T):
    if token_positions is None:
        return None
    if token_positions.shape != (B, Hkv, T):
        raise ValueError(f"token_positions.shape = {tuple(token_positions.shape)}, must be {(B, Hkv, T)}")
    if token_positions.dtype != torch.int32:
        token_positions = token_positions.to(torch.int32)
    if token_positions.stride(-1) != 1:
        token_positions = token_positions.contiguous()
    return token_positions


def prefill_core(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    scale: float,
    input_pos: int,
    token_positions: Optional[torch.Tensor] = None,
    return_weights: bool = False,
    return_lse: bool = False,
    output_transposed: bool = True,
    quant: Optional[QuantState] = None,
    num_splits: int = 0,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """Chunked-prefill attention on strided (B, H, len, D) views.

    Returns ``(out, weights, lse)``: ``out`` is (B, q, Hq, D) if ``output_transposed`` (the layout
    of the reference extension) else (B, Hq, q, D); ``weights`` fp32 (B, Hkv, T) summed over queries
    and averaged over the group; ``lse`` fp32 (B, q, Hq) in base 2."""
    _lib.require_gpu(query, key, value)
    for n, t in (("query", query), ("key", key), ("value", value)):
        _check_bhtd(n, t)
    _check_dtypes(query, key, value, quant)
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    if key.shape != value.shape or key.shape[0] != B or key.shape[3] != _row_len(D, key, quant):
        raise ValueError(f"key.shape = {tuple(key.shape)}, value.shape = {tuple(value.shape)} do not fit query {tuple(query.shape)}")
    if not (0 < q_len <= T):
        raise ValueError(f"Must have 0 < q_len = {q_len} <= kv_len = {T}")
    if Hkv <= 0 or Hq % Hkv != 0:
        raise ValueError(f"n_head = {Hq} must be a positive multiple of n_query_groups = {Hkv}")
    if D not in (ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES):
        raise NotImplementedError(f"head size {D} not in {ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES}")
    token_positions = _token_positions_i32(token_positions, B, Hkv, T)
    dev = query.device
    lib = _lib.load()
    with torch.cuda.device(dev):
        if output_transposed:
            out = torch.empty((B, q_len, Hq, D), dtype=query.dtype, device=dev)
            o_view = out.permute(0, 2, 1, 3)
        else:
            out = torch.empty((B, Hq, q_len, D), dtype=query.dtype, device=dev)
            o_view = out
        need_lse = return_lse or return_weights
        lse = torch.empty((B, q_len, Hq), dtype=torch.float32, device=dev) if need_lse else None
        w = torch.empty((B, Hkv, T), dtype=torch.float32, device=dev) if return_weights else None
        a = _lib.SdpaArgs()
        _fill_common(a, query, key, value, scale, input_pos, token_positions, quant, num_splits)
        a.o = o_view.data_ptr()
        a.o_stride_b, a.o_stride_h, a.o_stride_t = o_view.stride(0), o_view.stride(1), o_view.stride(2)
        a.lse = _lib.ptr(lse)
        a.w = _lib.ptr(w)
        nbytes = lib.kvx_sdpa_prefill_workspace_bytes(ctypes.byref(a))
        ws = _lib.workspace(dev, nbytes)
        a.workspace = _lib.ptr(ws)
        a.workspace_bytes = 0 if ws is None else ws.numel()
        fn = lib.kvx_sdpa_prefill_weights if return_weights else lib.kvx_sdpa_prefill
        _lib.check(fn(ctypes.byref(a), _lib.stream_ptr(dev)))
    return out, w, (lse if return_lse else None)


def score_sum_core(query, key, lse, scale, input_pos, token_positions=None, quant: Optional[QuantState] = None):
    """Score-sums from Q, K and a base-2 LSE (B, q, Hq): the stand-in for ``triton_score_sum``
    (keys_values/attention/flashinfer_wrapper.py:156-273) on strided (B, H, len, D) views."""
    _lib.require_gpu(query, key, lse)
    _check_bhtd("query", query)
    _check_bhtd("key", key)
    _check_dtypes(query, key, None, quant)
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    if lse.shape != (B, q_len, Hq) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError(f"lse must be contiguous float32 {(B, q_len, Hq)}, got {tuple(lse.shape)} {lse.dtype}")
    if D not in (ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES):
        raise NotImplementedError(f"head size {D} not in {ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES}")
    token_positions = _token_positions_i32(token_positions, B, Hkv, T)
    dev = query.device
    with torch.cuda.device(dev):
        w = torch.empty((B, Hkv, T), dtype=torch.float32, device=dev)
        a = _lib.SdpaArgs()
        if quant is not None:
            quant = QuantState(quant.k_scale, quant.k_zp, quant.k_scale, quant.k_zp)
        _fill_common(a, query, key, None, scale, input_pos, token_positions, quant, 0)
        a.lse = lse.data_ptr()
        a.w = w.data_ptr()
        lib = _lib.load()
        # short caches split the query rows over more workgroups; the partial sums need a workspace
        ws = _lib.workspace(dev, lib.kvx_sdpa_prefill_workspace_bytes(ctypes.byref(a)))
        a.workspace = _lib.ptr(ws)
        a.workspace_bytes = 0 if ws is None else ws.numel()
        _lib.check(lib.kvx_score_sum(ctypes.byref(a), _lib.stream_ptr(dev)))
    return w


def decode_core(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    scale: float,
    return_weights: bool = False,
    return_lse: bool = False,
    quant: Optional[QuantState] = None,
    num_splits: int = 0,
    scratch_splits: Optional[torch.Tensor] = None,
):
    """Single-token decode on strided views: query (B, Hq, 1, D), key/value (B, Hkv, T, D).
    Returns ``(out (B, Hq, D), weights (B, Hkv, T) or None, lse (B, 1, Hq) or None)``.
    ``scratch_splits``: optional one-element int32 device tensor that receives the number of KV splits whose logits
    went through the HBM scratch instead of staying on the chip (0 in the normal case)."""
    _lib.require_gpu(query, key, value)
    for n, t in (("query", query), ("key", key), ("value", value)):
        _check_bhtd(n, t)
    _check_dtypes(query, key, value, quant)
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    if q_len != 1:
        raise ValueError(f"decode needs q_len == 1, got {q_len}")
    if key.shape != value.shape or key.shape[0] != B or key.shape[3] != _row_len(D, key, quant):
        raise ValueError(f"key.shape = {tuple(key.shape)}, value.shape = {tuple(value.shape)} do not fit query {tuple(query.shape)}")
    if Hkv <= 0 or Hq % Hkv != 0:
        raise ValueError(f"n_head = {Hq} must be a positive multiple of n_query_groups = {Hkv}")
    if D not in (ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES):
        raise NotImplementedError(f"head size {D} not in {ALLOWED_HEAD_SIZES if quant is None else QUANTIZED_HEAD_SIZES}")
    dev = query.device
    lib = _lib.load()
    with torch.cuda.device(dev):
        out = torch.empty((B, Hq, D), dtype=query.dtype, device=dev)
        o_view = out.unsqueeze(2)
        w = torch.empty((B, Hkv, T), dtype=torch.float32, device=dev) if return_weights else None
        lse = torch.empty((B, 1, Hq), dtype=torch.float32, device=dev) if return_lse else None
        a = _lib.SdpaArgs()
        _fill_common(a, query, key, value, scale, max(T - 1, 0), None, quant, num_splits)
        a.o = o_view.data_ptr()
        a.o_stride_b, a.o_stride_h, a.o_stride_t = o_view.stride(0), o_view.stride(1), o_view.stride(2)
        a.w = _lib.ptr(w)
        a.lse = _lib.ptr(lse)
        if scratch_splits is not None:
            if scratch_splits.dtype != torch.int32 or scratch_splits.numel() != 1 or scratch_splits.device != dev:
                raise ValueError("scratch_splits must be a one-element int32 tensor on the query's device")
            a.decode_scratch_splits = scratch_splits.data_ptr()
        nbytes = lib.kvx_sdpa_decode_workspace_bytes(ctypes.byref(a))
        ws = _lib.workspace(dev, nbytes)
        a.workspace = _lib.ptr(ws)
        a.workspace_bytes = 0 if ws is None else ws.numel()
        _lib.check(lib.kvx_sdpa_decode(ctypes.byref(a), _lib.stream_ptr(dev)))
    return out, w, lse


# ---- the reference's entry points (keys_values/attention/flashinfer_ops.py:193-440) --------------


def _require_available():
    if not is_available():
        raise RuntimeError("keys_values_amd: libkvx.so is not built or no gfx950 device is visible")


def sdpa_decode(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    scale: float,
    return_weights: bool = False,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """As ``flashinfer_ops.sdpa_decode`` (keys_values/attention/flashinfer_ops.py:193-275):
    query [B, Hq, D] or [Hq, D]; key/value [B, T, Hkv, D] or [T, Hkv, D]. Returns the output in the
    shape of ``query`` and, if asked, fp32 weights [B, Hkv, T] (or [Hkv, T]) already divided by the
    group size."""
    _require_available()
    batched = query.ndim == 3
    if not batched:
        if query.ndim != 2 or key.ndim != 3:
            raise ValueError("query must be [B, Hq, D] or [Hq, D]; key/value [B, T, Hkv, D] or [T, Hkv, D]")
        query, key, value = query.unsqueeze(0), key.unsqueeze(0), value.unsqueeze(0)
    if key.ndim != 4 or value.ndim != 4:
        raise ValueError("key and value must be [B, T, Hkv, D]")
    out, w, _ = decode_core(query.unsqueeze(2), key.permute(0, 2, 1, 3), value.permute(0, 2, 1, 3), scale, return_weights)
    if not batched:
        out = out.squeeze(0)
        w = None if w is None else w.squeeze(0)
    return out, w


def sdpa_prefill(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    scale: float,
    return_weights: bool = False,
    return_lse: bool = False,
    token_positions: Optional[torch.Tensor] = None,
    input_pos: Optional[int] = None,
) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[torch.Tensor]]:
    """As ``flashinfer_ops.sdpa_prefill`` (keys_values/attention/flashinfer_ops.py:278-354):
    query [B, q, Hq, D] (or [q, Hq, D]), key/value [B, T, Hkv, D]; right-aligned causal mask unless
    ``token_positions`` [B, Hkv, T] and ``input_pos`` say otherwise. Returns
    ``(out [B, q, Hq, D], weights [B, Hkv, T] or None, lse [B, q, Hq] base 2 or None)``."""
    _require_available()
    batched = query.ndim == 4
    if not batched:
        if query.ndim != 3 or key.ndim != 3:
            raise ValueError("query must be [B, q, Hq, D] or [q, Hq, D]")
        query, key, value = query.unsqueeze(0), key.unsqueeze(0), value.unsqueeze(0)
        if token_positions is not None:
            token_positions = token_positions.unsqueeze(0)
    if key.ndim != 4 or value.ndim != 4:
        raise ValueError("key and value must be [B, T, Hkv, D]")
    q_len, T = query.shape[1], key.shape[1]
    if input_pos is None:
        input_pos = T - q_len
    out, w, lse = prefill_core(
        query.permute(0, 2, 1, 3), key.permute(0, 2, 1, 3), value.permute(0, 2, 1, 3), scale, input_pos,
        token_positions, return_weights, return_lse, output_transposed=True,
    )
    if not batched:
        out = out.squeeze(0)
        w = None if w is None else w.squeeze(0)
        lse = None if lse is None else lse.squeeze(0)
    return out, w, lse


# The reference keeps two more spellings of the weights-returning prefill
# (keys_values/attention/flashinfer_ops.py:357-440); here they are the same two-kernel path.
sdpa_prefill_fused = sdpa_prefill
sdpa_prefill_fused_v2 = sdpa_prefill


def default_scale(head_size: int) -> float:
    return 1.0 / math.sqrt(head_size)
