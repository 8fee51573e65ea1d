"""
K/V buffer objects with the surface of ``KVCacheBuffers`` / ``DefaultKVCacheBuffers``
(keys_values/kvcache/buffers.py:134-551) and the holder types that cross from the cache to the attention
operator, ``KeysAndValues`` / ``DefaultKeysAndValues`` (keys_values/attention/base.py:46-93), on the HIP
kernels. A cache class written against the reference's buffer interface (its ``AttnWeightsKVCache`` keeps
positions and scores itself and only calls ``forward``, ``prefill``, ``get_slots``, ``set_slots``,
``get_keys_values``, ``write_back``) can sit on these buffers unchanged.

``HipKVCacheBuffers`` holds ``k`` / ``v`` of shape ``(batch, n_query_groups, cache_length, head_size)`` as
bfloat16 or float16 rows, or as 8-bit / 4-bit codes with per-row scale and zero point (the store of
``QuantizedKVCacheBuffers`` with a ``TorchBasicQuantizer``, keys_values/kvcache/quant_buffers.py:361-804,
without its dequantised working copy: the codes stay resident, rows are quantised when written and
``write_back`` has nothing left to do). Slot writes go through ``kvx_cache_write``; there is no CPU path.
With ``blocks_over_heads=True`` the quantisation blocks are the slots over all heads, held by two
``RowQuantizer`` stores and served by the quantiser's block kernels.
"""
import ctypes
from dataclasses import dataclass
from typing import Dict, Optional, Tuple, Union

import torch

from .. import _lib
from ..attention import ops
from .quantize import RowQuantizer

PositionsType = Union[torch.Tensor, Tuple[int, int]]


class KeysAndValues:
    """keys_values/attention/base.py:46-70: what the cache hands to the attention operator."""

    def keys(self) -> torch.Tensor:
        raise NotImplementedError()

    def values(self) -> torch.Tensor:
        raise NotImplementedError()


class DefaultKeysAndValues(KeysAndValues):
    """keys_values/attention/base.py:73-93."""

    def __init__(self, keys: torch.Tensor, values: torch.Tensor):
        if keys.ndim != 4 or keys.shape[:-1] != values.shape[:-1]:
            raise ValueError(f"keys {tuple(keys.shape)} and values {tuple(values.shape)} must be 4D and agree up to the last axis")
        self._keys = keys
        self._values = values

    def keys(self) -> torch.Tensor:
        return self._keys

    def values(self) -> torch.Tensor:
        return self._values

    def clear(self):
        self._keys = None
        self._values = None


class QuantizedKeysAndValues(KeysAndValues):
    """Views of a quantised store: ``key_codes`` / ``value_codes`` (uint8, D or D/2 bytes per row) with
    ``quant`` (``ops.QuantState``) are what the attention kernels read in place; ``keys()`` / ``values()``
    dequantise into new tensors for any other consumer, as the reference's
    ``DequantizedBufferKeysAndValues`` does (keys_values/kvcache/quant_buffers.py:807-833)."""

    def __init__(self, key_codes: torch.Tensor, value_codes: torch.Tensor, quant: ops.QuantState, head_size: int, num_bits: int,
                 dtype: torch.dtype = torch.bfloat16):
        self.key_codes, self.value_codes, self.quant = key_codes, value_codes, quant
        self.head_size, self.num_bits, self.dtype = head_size, num_bits, dtype

    def _dequantize(self, codes, scale, zp) -> torch.Tensor:
        b, h, t, _ = codes.shape
        out = torch.empty((b, h, t, self.head_size), dtype=self.dtype, device=codes.device)
        _dequantize_rows(codes, scale, zp, out, self.num_bits)
        return out

    def keys(self) -> torch.Tensor:
        return self._dequantize(self.key_codes, self.quant.k_scale, self.quant.k_zp)

    def values(self) -> torch.Tensor:
        return self._dequantize(self.value_codes, self.quant.v_scale, self.quant.v_zp)


def _dequantize_rows(codes, scale, zp, out, num_bits: int):
    """codes (b, h, t, row bytes) strided over t only at the slot axis, state (b, h, t), out (b, h, t, D)
    contiguous: one launch per (b, h) run of contiguous slots."""
    lib = _lib.load()
    elem = _lib.elem_kv_dtype(out.dtype)

    def fn(c, s, z, rows, dd, o, stride, stream):  # the rows dequantise to the type of `out`
        return lib.kvx_dequantize_rows_typed(c, s, z, rows, dd, num_bits, elem, o, stride, stream)

    b, h, t, row = codes.shape
    d = out.shape[-1]
    dev = codes.device
    with torch.cuda.device(dev):
        st = _lib.stream_ptr(dev)
        if codes.is_contiguous() and scale.is_contiguous() and zp.is_contiguous():
            _lib.check(fn(codes.data_ptr(), scale.data_ptr(), zp.data_ptr(), b * h * t, d, out.data_ptr(), d, st))
            return
        if codes.stride(2) != row or codes.stride(3) != 1 or scale.stride(2) != 1 or zp.stride(2) != 1:
            codes, scale, zp = codes.contiguous(), scale.contiguous(), zp.contiguous()
            _lib.check(fn(codes.data_ptr(), scale.data_ptr(), zp.data_ptr(), b * h * t, d, out.data_ptr(), d, st))
            return
        for bi in range(b):  # slot runs of a cache view: contiguous per (batch, head)
            for hi in range(h):
                _lib.check(fn(codes[bi, hi].data_ptr(), scale[bi, hi].data_ptr(), zp[bi, hi].data_ptr(), t, d, out[bi, hi].data_ptr(), d, st))


@dataclass(frozen=True)
class KVCacheBuffersParams:
    """keys_values/kvcache/buffers.py:31-74."""

    max_batch_size: int
    n_query_groups: int
    head_size: int
    device: Optional[torch.device] = None
    dtype: Optional[torch.dtype] = None

    @staticmethod
    def from_params(cache_params) -> "KVCacheBuffersParams":
        return KVCacheBuffersParams(cache_params.max_batch_size, cache_params.n_query_groups, cache_params.head_size, None, cache_params.dtype)


class KVCacheBuffers:
    """The interface, keys_values/kvcache/buffers.py:134-401."""

    def __init__(self, params: KVCacheBuffersParams, cache_length: int):
        self.max_batch_size = params.max_batch_size
        self.n_query_groups = params.n_query_groups
        self.cache_length = cache_length
        self.head_size = params.head_size
        self.dtype = params.dtype
        self.batch_size = None
        self.current_length = None

    def forward(self, positions: PositionsType, key: torch.Tensor, value: torch.Tensor) -> KeysAndValues:
        """Write ``key`` / ``value`` to the slots ``positions``, return the buffers up to the current length
        (keys_values/kvcache/buffers.py:231-262)."""
        if self.batch_size is None or self.current_length is None:
            raise IndexError("Buffers are not initialised, call 'prefill' first")
        num = key.shape[2]
        self.current_length = min(self.cache_length, self.current_length + num)
        return self._forward(positions, key, value)

    def prefill(self, key: torch.Tensor, value: torch.Tensor):
        self.batch_size, self.current_length = self._check_prefill(key, value)
        self._prefill(key, value)

    def _check_prefill(self, key: torch.Tensor, value: Optional[torch.Tensor]) -> Tuple[int, int]:
        """keys_values/kvcache/buffers.py:295-311."""
        if key.dim() != 4:
            raise ValueError("key must have 4 dimensions")
        batch_size, _, init_length, _ = key.shape
        if not (1 <= batch_size <= self.max_batch_size):
            raise ValueError(f"key.shape[0] = {batch_size} must be in [1, {self.max_batch_size}]")
        shape = (batch_size, self.n_query_groups, init_length, self.head_size)
        if tuple(key.shape) != shape or (value is not None and tuple(value.shape) != shape):
            raise ValueError(f"Shapes of key, value must be {shape}, but key.shape = {tuple(key.shape)}"
                             + (f", value.shape = {tuple(value.shape)}" if value is not None else ""))
        return batch_size, init_length

    def write_back(self):
        pass

    def reset(self):
        self.current_length = 0

    def deallocate(self):
        self._deallocate()
        self.reset()

    def get_params(self) -> KVCacheBuffersParams:
        return KVCacheBuffersParams(self.max_batch_size, self.n_query_groups, self.head_size, self.device, self.dtype)


_STORE_BITS = {"default": None, "torch-quantized8": 8, "torch-quantized4": 4}


class BlockQuantizedKeysAndValues(KeysAndValues):
    """The first ``length`` slots of a store whose quantisation blocks run over the heads, dequantised on demand."""

    def __init__(self, quantizer_k, quantizer_v, batch_size: int, length: int):
        self._qk, self._qv, self._b, self._t = quantizer_k, quantizer_v, batch_size, length

    def keys(self) -> torch.Tensor:
        return self._qk.dequantize(0, self._t)[: self._b]

    def values(self) -> torch.Tensor:
        return self._qv.dequantize(0, self._t)[: self._b]


class HipKVCacheBuffers(KVCacheBuffers):
    def __init__(self, params: KVCacheBuffersParams, cache_length: int, allocate_buffers: bool = False, num_bits: Optional[int] = None,
                 blocks_over_heads: bool = False):
        """``num_bits``: None for plain rows, 8 or 4 for the quantised store. ``blocks_over_heads``: one quantisation
        block per slot over all heads (keys_values/kvcache/quant_buffers.py:849-870) instead of one per (head, slot)
        row; ignored by the plain store. A slot written for some heads only is requantised as a whole from the
        dequantised rows of the others, as the reference's write-back of its dequantised working buffer does
        (keys_values/kvcache/quant_buffers.py:368-375). This form is served by the block kernels of the quantiser;
        the attention kernels read the one-block-per-row store only, so a cache on top of it attends over the rows
        that ``get_keys_values`` dequantises."""
        super().__init__(params, cache_length)
        if num_bits not in (None, 4, 8):
            raise ValueError(f"num_bits = {num_bits}, must be None, 4 or 8")
        self.blocks_over_heads = bool(blocks_over_heads) and num_bits is not None
        self._qk = self._qv = None  # the two block stores (blocks over the heads only)
        sizes = ops.ALLOWED_HEAD_SIZES if num_bits is None else ops.QUANTIZED_HEAD_SIZES
        if params.head_size not in sizes:
            raise NotImplementedError(f"head_size = {params.head_size} not in {sizes}")
        if self.dtype is not None and self.dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"dtype {self.dtype}: the kernels take bfloat16 or float16 rows")
        self.num_bits = num_bits
        self.k = self.v = None
        self.k_scale = self.k_zp = self.v_scale = self.v_zp = None
        self._device = torch.device(params.device) if params.device is not None else None
        if allocate_buffers:
            self._allocate_buffers(self._device)

    # -- allocation (keys_values/kvcache/buffers.py:426-478) -----------------------------------------------

    @property
    def device(self) -> Optional[torch.device]:
        return None if self.k is None else self.k.device

    @property
    def buffers_are_allocated(self) -> bool:
        return self.k is not None

    @property
    def quantized(self) -> bool:
        return self.num_bits is not None

    def _row_bytes(self) -> int:
        return self.head_size // 2 if self.num_bits == 4 else self.head_size

    def _allocate_buffers(self, device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None):
        if device is None:
            device = self.device if self.buffers_are_allocated else torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError(f"HipKVCacheBuffers live on a ROCm device, not on {device}: there is no CPU path")
        if self.dtype is None:
            if dtype not in (torch.bfloat16, torch.float16):
                raise NotImplementedError(f"dtype {dtype} is not served by this store")
            self.dtype = dtype
        batch_size = self.batch_size
        if not self.buffers_are_allocated:
            batch_size = self.max_batch_size if batch_size is None else batch_size
        elif batch_size is not None and self.k.shape[0] >= batch_size and device == self.device:
            batch_size = None  # large enough already
        if batch_size is None:
            return
        b, h, length = batch_size, self.n_query_groups, self.cache_length
        if self.blocks_over_heads:
            shape = (b, h, length, self.head_size)
            self._qk = RowQuantizer(shape, self.dtype, self.num_bits, True, allocate_buffers=True, device=device)
            self._qv = RowQuantizer(shape, self.dtype, self.num_bits, True, allocate_buffers=True, device=device)
            for q in (self._qk, self._qv):
                q.quant_buffer.zero_()
            # the same names as the row store; shapes (b, length, h * row bytes) and (b, length)
            self.k, self.v = self._qk.quant_buffer, self._qv.quant_buffer
            self.k_scale, self.v_scale = self._qk.quant_scales, self._qv.quant_scales
            self.k_zp, self.v_zp = self._qk.quant_zero_points, self._qv.quant_zero_points
        elif self.quantized:
            self.k = torch.zeros((b, h, length, self._row_bytes()), dtype=torch.uint8, device=device)
            self.v = torch.zeros_like(self.k)
            self.k_scale = torch.zeros((b, h, length), dtype=torch.float32, device=device)
            self.v_scale = torch.zeros_like(self.k_scale)
            self.k_zp = torch.zeros((b, h, length), dtype=torch.int32, device=device)
            self.v_zp = torch.zeros_like(self.k_zp)
        else:
            self.k = torch.zeros((b, h, length, self.head_size), dtype=self.dtype, device=device)
            self.v = torch.zeros_like(self.k)

    def _deallocate(self):
        self.k = self.v = None
        self._qk = self._qv = None
        self.k_scale = self.k_zp = self.v_scale = self.v_zp = None

    def _require_buffers(self):
        if not self.buffers_are_allocated:
            raise IndexError("Buffers are not allocated. Call 'prefill' first")
        if self.batch_size is None or self.current_length is None:
            raise IndexError("Buffers are not initialised, call 'prefill' first")

    # -- slots (keys_values/kvcache/buffers.py:482-551) ----------------------------------------------------

    def _check_positions(self, positions: PositionsType, num: Optional[int] = None) -> torch.Tensor:
        """Slot positions as an int32 (batch, n_query_groups, num) device tensor."""
        if isinstance(positions, torch.Tensor):
            shape = (self.batch_size, self.n_query_groups)
            if positions.ndim != 3 or tuple(positions.shape[:2]) != shape or (num is not None and positions.shape[2] != num):
                raise ValueError(f"positions.shape = {tuple(positions.shape)}, must be {shape + (num if num is not None else 'num',)}")
            idx = positions.to(device=self.device, dtype=torch.int32)
            return idx if idx.stride(-1) == 1 else idx.contiguous()
        start, end = positions
        if not (0 <= start < end <= self.cache_length) or (num is not None and end - start != num):
            raise ValueError(f"positions = {positions} must be a range inside [0, {self.cache_length}]" + (f" of {num} slots" if num is not None else ""))
        return torch.arange(start, end, dtype=torch.int32, device=self.device).view(1, 1, -1).expand(self.batch_size, self.n_query_groups, -1).contiguous()

    def _quant_state(self, t: int) -> Optional[ops.QuantState]:
        if not self.quantized:
            return None
        b = self.batch_size
        return ops.QuantState(self.k_scale[:b, :, :t], self.k_zp[:b, :, :t], self.v_scale[:b, :, :t], self.v_zp[:b, :, :t])

    def set_slots(self, positions: PositionsType, key: torch.Tensor, value: torch.Tensor):
        self._require_buffers()
        b, h, num, d = key.shape
        if (b, h, d) != (self.batch_size, self.n_query_groups, self.head_size) or key.shape != value.shape:
            raise ValueError(f"key.shape = {tuple(key.shape)}, value.shape = {tuple(value.shape)} do not fit the buffers")
        if self.blocks_over_heads:
            if not isinstance(positions, torch.Tensor):
                self._check_positions(positions, num)
            return self._set_block_slots(positions, key.to(device=self.device, dtype=self.dtype), value.to(device=self.device, dtype=self.dtype))
        index = self._check_positions(positions, num)
        key = key.to(device=self.device, dtype=self.dtype)
        value = value.to(device=self.device, dtype=self.dtype)
        if key.stride(-1) != 1:
            key = key.contiguous()
        if value.stride(-1) != 1:
            value = value.contiguous()
        a = _lib.CacheWriteArgs()
        a.B, a.Hkv, a.num, a.D, a.cache_len = b, h, num, d, self.cache_length
        a.kv_dtype = _lib.elem_kv_dtype(self.dtype) if self.num_bits is None else _lib.quant_kv_dtype(self.num_bits, self.dtype)
        a.index, a.index_stride_b, a.index_stride_h = index.data_ptr(), index.stride(0), index.stride(1)
        a.key, a.key_stride_b, a.key_stride_h, a.key_stride_t = key.data_ptr(), key.stride(0), key.stride(1), key.stride(2)
        a.value, a.value_stride_b, a.value_stride_h, a.value_stride_t = value.data_ptr(), value.stride(0), value.stride(1), value.stride(2)
        a.k_cache, a.kc_stride_b, a.kc_stride_h, a.kc_stride_t = self.k.data_ptr(), self.k.stride(0), self.k.stride(1), self.k.stride(2)
        a.v_cache, a.vc_stride_b, a.vc_stride_h, a.vc_stride_t = self.v.data_ptr(), self.v.stride(0), self.v.stride(1), self.v.stride(2)
        if self.quantized:
            a.k_scale, a.k_zp, a.v_scale, a.v_zp = self.k_scale.data_ptr(), self.k_zp.data_ptr(), self.v_scale.data_ptr(), self.v_zp.data_ptr()
            a.qs_stride_b, a.qs_stride_h = self.k_scale.stride(0), self.k_scale.stride(1)
        # rows only: positions, scores and the ring are the cache's business (token_pos = NULL)
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().kvx_cache_write(ctypes.byref(a), _lib.stream_ptr(self.device)))

    # -- blocks over the heads ------------------------------------------------------------------------------

    def _gathered(self, q: "RowQuantizer", blocks: torch.Tensor) -> "RowQuantizer":
        """A scratch store holding copies of the blocks ``blocks`` (flat batch * cache_length + slot indices)."""
        n = blocks.numel()
        tmp = RowQuantizer((1, self.n_query_groups, n, self.head_size), self.dtype, self.num_bits, True, allocate_buffers=True, device=self.device)
        tmp.quant_buffer[0] = q.quant_buffer.view(-1, q.quant_buffer.shape[-1])[blocks]
        tmp.quant_scales[0] = q.quant_scales.view(-1)[blocks]
        tmp.quant_zero_points[0] = q.quant_zero_points.view(-1)[blocks]
        return tmp

    def _flat_blocks(self, index: torch.Tensor) -> torch.Tensor:
        b = index.shape[0]
        return (torch.arange(b, device=index.device).view(b, 1, 1) * self.cache_length + index.long()).reshape(-1)

    def _set_block_slots(self, positions: PositionsType, key: torch.Tensor, value: torch.Tensor):
        b, h, num, d = key.shape
        for q in (self._qk, self._qv):
            q.allocate_buffers(b)  # the batch size of this fill
        if not isinstance(positions, torch.Tensor):  # every head writes the same slots: whole blocks are replaced
            self._qk.quantize(positions[0], positions[1], key)
            self._qv.quantize(positions[0], positions[1], value)
            return
        index = self._check_positions(positions, num)
        blocks, where = torch.unique(self._flat_blocks(index), return_inverse=True)
        heads = torch.arange(h, device=self.device).view(1, h, 1).expand(b, h, num).reshape(-1)
        for q, new in ((self._qk, key), (self._qv, value)):
            tmp = self._gathered(q, blocks)
            rows = tmp.dequantize(0, blocks.numel())  # (1, h, n, d): the other heads' rows as the store holds them
            rows[0, heads, where] = new.reshape(-1, d)
            tmp.quantize(0, blocks.numel(), rows)
            q.quant_buffer.view(-1, q.quant_buffer.shape[-1])[blocks] = tmp.quant_buffer[0]
            q.quant_scales.view(-1)[blocks] = tmp.quant_scales[0]
            q.quant_zero_points.view(-1)[blocks] = tmp.quant_zero_points[0]

    def _get_block_slots(self, positions: PositionsType) -> Tuple[torch.Tensor, torch.Tensor]:
        b, h = self.batch_size, self.n_query_groups
        if not isinstance(positions, torch.Tensor):
            start, end = positions
            if not (0 <= start < end <= self.cache_length):
                raise ValueError(f"positions = {positions} must be a range inside [0, {self.cache_length}]")
            return self._qk.dequantize(start, end)[:b], self._qv.dequantize(start, end)[:b]
        index = self._check_positions(positions)
        num = index.shape[2]
        blocks = self._flat_blocks(index)  # one block per (batch, head, position): the head's row is picked below
        heads = torch.arange(h, device=self.device).view(1, h, 1).expand(b, h, num).reshape(-1)
        each = torch.arange(blocks.numel(), device=self.device)
        out = []
        for q in (self._qk, self._qv):
            rows = self._gathered(q, blocks).dequantize(0, blocks.numel())
            out.append(rows[0, heads, each].view(b, h, num, self.head_size))
        return out[0], out[1]

    def get_slots(self, positions: PositionsType) -> Tuple[torch.Tensor, torch.Tensor]:
        self._require_buffers()
        if self.blocks_over_heads:
            return self._get_block_slots(positions)
        b = self.batch_size
        if isinstance(positions, torch.Tensor):
            index = self._check_positions(positions).to(torch.int64)
            gi = index.unsqueeze(-1).expand(-1, -1, -1, self.k.shape[-1])
            kk, vv = self.k[:b].gather(-2, gi), self.v[:b].gather(-2, gi)
            if not self.quantized:
                return kk, vv
            st = [t[:b].gather(-1, index) for t in (self.k_scale, self.k_zp, self.v_scale, self.v_zp)]
        else:
            start, end = positions
            if not (0 <= start < end <= self.cache_length):
                raise ValueError(f"positions = {positions} must be a range inside [0, {self.cache_length}]")
            kk, vv = self.k[:b, :, start:end], self.v[:b, :, start:end]
            if not self.quantized:
                return kk, vv
            st = [t[:b, :, start:end] for t in (self.k_scale, self.k_zp, self.v_scale, self.v_zp)]
        kv = QuantizedKeysAndValues(kk, vv, ops.QuantState(*st), self.head_size, self.num_bits, self.dtype)
        return kv.keys(), kv.values()

    def _forward(self, positions: PositionsType, key: torch.Tensor, value: torch.Tensor) -> KeysAndValues:
        self.set_slots(positions, key, value)
        return self.get_keys_values()

    def get_keys_values(self) -> Optional[KeysAndValues]:
        if not self.buffers_are_allocated or self.batch_size is None or self.current_length is None:
            return None
        b, t = self.batch_size, self.current_length
        if self.blocks_over_heads:
            return BlockQuantizedKeysAndValues(self._qk, self._qv, b, t)
        if not self.quantized:
            return DefaultKeysAndValues(self.k[:b, :, :t], self.v[:b, :, :t])
        return QuantizedKeysAndValues(self.k[:b, :, :t], self.v[:b, :, :t], self._quant_state(t), self.head_size, self.num_bits, self.dtype)

    def _prefill(self, key: torch.Tensor, value: torch.Tensor):
        if self.buffers_are_allocated and key.device != self.device:
            raise ValueError(f"key.device = {key.device}, must be {self.device}")
        _lib.require_gpu(key, value)
        self._allocate_buffers(device=key.device, dtype=key.dtype)
        self.set_slots((0, key.shape[2]), key, value)

    def prefill_from_keys_values(self, k_and_v: KeysAndValues):
        """keys_values/kvcache/buffers.py:553-575: only the first ``cache_length`` slots are taken."""
        keys = k_and_v.keys()
        self.batch_size, init_length = self._check_prefill(keys, None)
        init_length = min(init_length, self.cache_length)
        self.current_length = init_length
        self._prefill(keys[:, :, :init_length], k_and_v.values()[:, :, :init_length])

    # -- sizes (keys_values/kvcache/buffers.py:577-612) ------------------------------------------------------

    def size_estimate(self) -> Tuple[int, Dict[str, int]]:
        self._require_buffers()
        parts = {"buffers": 8 * (self.k.numel() * self.k.element_size() + self.v.numel() * self.v.element_size())}
        if self.quantized:
            parts["quant_state"] = 8 * sum(t.numel() * t.element_size() for t in (self.k_scale, self.k_zp, self.v_scale, self.v_zp))
        return sum(parts.values()), parts

    @staticmethod
    def size_estimate_apriori(params: KVCacheBuffersParams, **kwargs) -> Tuple[int, Dict[str, int]]:
        cache_length = kwargs.get("cache_length")
        if cache_length is None:
            raise IndexError("Argument 'cache_length' is missing")
        num_bits = kwargs.get("num_bits")
        rows = params.max_batch_size * params.n_query_groups * int(cache_length)
        states = params.max_batch_size * int(cache_length) if kwargs.get("blocks_over_heads") else rows  # scale + zero point each
        if num_bits is None:
            if params.dtype is None:
                raise ValueError("params.dtype must be provided")
            parts = {"buffers": 2 * rows * params.head_size * 8 * torch.empty((), dtype=params.dtype).element_size()}
        else:
            parts = {"buffers": 2 * rows * params.head_size * num_bits, "quant_state": 2 * states * 64}
        return sum(parts.values()), parts


def create_kv_cache_buffers(store: str, params: KVCacheBuffersParams, cache_length: int, **kwargs) -> HipKVCacheBuffers:
    """``default``, ``torch-quantized8`` or ``torch-quantized4``: the buffer part of the reference's cache
    names (keys_values/kvcache/factory.py:50-66)."""
    if store not in _STORE_BITS:
        raise NotImplementedError(f"store '{store}' must be one of {sorted(_STORE_BITS)}")
    return HipKVCacheBuffers(params, cache_length, num_bits=_STORE_BITS[store], **kwargs)
