"""
``RowQuantizer``: ``TorchBasicQuantizer`` (keys_values/kvcache/quantize/pytorch.py:157-564) on the HIP
kernels: 8-bit or 4-bit affine min-max codes, one quantisation block per (token, head) row or, with
``blocks_over_heads=True``, per token over all heads. Same buffer names, shapes and dtypes
(``quant_buffer`` uint8 ``(first, L, final)``, ``quant_scales`` float32 ``(first, L)``,
``quant_zero_points`` int32 ``(first, L)`` with ``first = B*Hkv, final = D[/2]`` or
``first = B, final = Hkv*D[/2]``, :235-245,281-295), same methods with the same meaning
(``allocate_buffers``, ``deallocate``, ``quantize``, ``dequantize``, ``quantization_error``;
keys_values/kvcache/quantize/quantization.py:102-236). Codes, scales and zero points are
bit-identical to the reference's for every block whose zero point fits int32. The 4-bit store packs
two codes per byte, the first half of the block in the high nibbles (:384-393,457-465).

``RowQuantizer8`` is the 8-bit, one-block-per-row case under its earlier name.
"""
import ctypes
from typing import Optional, Tuple

import torch

from .. import _lib


class RowQuantizer:
    def __init__(
        self,
        shape: Tuple[int, int, int, int],
        source_dtype: torch.dtype = torch.bfloat16,
        num_bits: int = 8,
        blocks_over_heads: bool = False,
        allocate_buffers: bool = False,
        device: Optional[torch.device] = None,
    ):
        if len(shape) != 4 or any(x < 1 for x in shape):
            raise ValueError(f"shape = {shape}, must be 4D and all positive")
        if num_bits not in (4, 8):  # keys_values/kvcache/quantize/pytorch.py:191-192
            raise ValueError(f"num_bits = {num_bits}, must be 4 or 8")
        if source_dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"source_dtype = {source_dtype}: the kernels take bfloat16 or float16 rows")
        if shape[3] % 16 != 0:
            raise NotImplementedError(f"head_size = {shape[3]} must be a multiple of 16")
        self.shape = tuple(shape)
        self.source_dtype = source_dtype
        self.num_bits = num_bits
        self.blocks_over_heads = blocks_over_heads
        self.max_batch_size, self.n_query_groups = shape[0], shape[1]
        self.blocksize = shape[1] * shape[3] if blocks_over_heads else shape[3]
        if self.blocksize > 8192:
            raise NotImplementedError(f"blocksize = {self.blocksize} exceeds the 8192 values of one quantisation block")
        self.quant_buffer = None
        self.quant_scales = None
        self.quant_zero_points = None
        self._batch_size = None
        if allocate_buffers:
            self.allocate_buffers(shape[0], device)

    # -- buffers (keys_values/kvcache/quantize/pytorch.py:231-310) ---------------------------------

    @property
    def device(self) -> Optional[torch.device]:
        return self.quant_buffer.device if self.quant_buffer is not None else None

    @property
    def batch_size(self) -> Optional[int]:
        return self._batch_size

    @property
    def buffers_are_allocated(self) -> bool:
        return self.quant_buffer is not None

    def _quant_shape(self, batch_size: int) -> Tuple[int, int, int]:
        _, hkv, length, _ = self.shape
        first = batch_size if self.blocks_over_heads else batch_size * hkv
        return first, length, self.blocksize * self.num_bits // 8

    def allocate_buffers(self, batch_size: int, device: Optional[torch.device] = None):
        if not (0 < batch_size <= self.max_batch_size):
            raise ValueError(f"batch_size = {batch_size} must be in (0, {self.max_batch_size}]")
        if device is None:
            device = self.device if self.buffers_are_allocated else torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError(f"RowQuantizer buffers live on a ROCm device, not on {device}: there is no CPU path")
        if (not self.buffers_are_allocated) or batch_size > self.shape[0] or device != self.device:
            self.shape = (batch_size,) + self.shape[1:]
            qs = self._quant_shape(batch_size)
            self.quant_buffer = torch.empty(qs, dtype=torch.uint8, device=device)
            self.quant_scales = torch.zeros(qs[:-1], dtype=torch.float32, device=device)
            self.quant_zero_points = torch.zeros(qs[:-1], dtype=torch.int32, device=device)
        self._batch_size = batch_size

    def deallocate(self):
        self.quant_buffer = None
        self.quant_scales = None
        self.quant_zero_points = None
        self._batch_size = None

    # -- quantise / dequantise -----------------------------------------------------------------------

    def _block_args(self, x: torch.Tensor, start: int, buffer, scales, zps) -> _lib.BlockQuantArgs:
        """x (B, Hkv, num, D) bf16 with D contiguous; blocks land in slots start.. of the buffers."""
        b, hkv, num, d = x.shape
        a = _lib.BlockQuantArgs()
        a.x = x.data_ptr()
        if self.blocks_over_heads:  # block (b, t): all heads of a token
            a.n_outer, a.n_inner, a.nseg = b, num, hkv
            a.x_stride_outer, a.x_stride_inner, a.x_stride_seg = x.stride(0), x.stride(2), x.stride(1)
        else:  # block (b * Hkv + h, t)
            a.n_outer, a.n_inner, a.nseg = b * hkv, num, 1
            a.x_stride_outer, a.x_stride_inner, a.x_stride_seg = x.stride(1), x.stride(2), 0
        a.D, a.bits, a.elem_dtype = d, self.num_bits, _lib.elem_kv_dtype(self.source_dtype)
        a.codes = buffer[0, start].data_ptr()
        a.codes_stride_outer = buffer.stride(0)
        a.scale, a.zp = scales[0, start:].data_ptr(), zps[0, start:].data_ptr()
        a.state_stride_outer = scales.stride(0)
        return a

    def _kernel_view(self, x: torch.Tensor) -> torch.Tensor:
        """A view (or copy) of x the block kernels can address: rows 16-byte aligned, strides multiples
        of 8 and, for one block per row, the (batch, head) axes collapsible into one."""
        ok = x.stride(-1) == 1 and x.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in x.stride()[:3])
        if ok and not self.blocks_over_heads and x.shape[0] > 1:
            ok = x.stride(0) == x.shape[1] * x.stride(1)
        return x if ok else x.contiguous()

    def quantize(self, start: int, end: int, values: torch.Tensor, block_idx: Optional[int] = None):
        """Quantise slots ``range(start, end)`` from ``values`` (B, Hkv, end - start, D)
        (keys_values/kvcache/quantize/pytorch.py:312-355)."""
        if not self.buffers_are_allocated:
            raise IndexError("Quantizer buffers are not allocated")
        if self.batch_size != values.shape[0]:
            raise ValueError(f"batch_size = {self.batch_size}, values.shape[0] = {values.shape[0]}. Must be equal.")
        b, hkv, length, d = self._batch_size, self.shape[1], self.shape[2], self.shape[3]
        num = end - start
        if not (0 <= start <= end <= length) or tuple(values.shape) != (b, hkv, num, d):
            raise ValueError(f"values.shape = {tuple(values.shape)}, must be {(b, hkv, num, d)} with 0 <= start <= end <= {length}")
        if num == 0:
            return
        _lib.require_gpu(values)
        values = values.to(self.source_dtype)
        lib = _lib.load()
        dev = self.device
        with torch.cuda.device(dev):
            st = _lib.stream_ptr(dev)
            if not self.blocks_over_heads and d in (64, 128, 256) and start == 0 and end == length and values.is_contiguous():
                # the whole store in one pass of the row kernels (16 or 8 lanes per row)
                _lib.check(lib.kvx_quantize_rows_typed(values.data_ptr(), d, b * hkv * length, d, self.num_bits,
                                                       _lib.elem_kv_dtype(self.source_dtype), self.quant_buffer.data_ptr(),
                                                       self.quant_scales.data_ptr(), self.quant_zero_points.data_ptr(), st))
                return
            x = self._kernel_view(values)
            a = self._block_args(x, start, self.quant_buffer, self.quant_scales, self.quant_zero_points)
            _lib.check(lib.kvx_quantize_blocks(ctypes.byref(a), st))

    def dequantize(self, start: int, end: int, out: Optional[torch.Tensor] = None, block_idx: Optional[int] = None):
        """Dequantise slots ``range(start, end)`` to (B, Hkv, end - start, D) in the source dtype
        (keys_values/kvcache/quantize/pytorch.py:411-455)."""
        if not self.buffers_are_allocated:
            raise IndexError("Quantizer buffers are not allocated")
        b, hkv, length, d = self._batch_size, self.shape[1], self.shape[2], self.shape[3]
        num = end - start
        if not (0 <= start <= end <= length):
            raise ValueError(f"need 0 <= start <= end <= {length}")
        dev = self.device
        if out is None:
            out = torch.empty((b, hkv, num, d), dtype=self.source_dtype, device=dev)
        elif tuple(out.shape) != (b, hkv, num, d) or out.dtype != self.source_dtype or not out.is_contiguous():
            raise ValueError(f"out must be contiguous {self.source_dtype} of shape {(b, hkv, num, d)}")
        if num == 0:
            return out
        lib = _lib.load()
        with torch.cuda.device(dev):
            a = self._block_args(out, start, self.quant_buffer, self.quant_scales, self.quant_zero_points)
            _lib.check(lib.kvx_dequantize_blocks(ctypes.byref(a), _lib.stream_ptr(dev)))
        return out

    def quantization_error(self, x: torch.Tensor) -> torch.Tensor:
        """Per-row L2 norm of ``x - dequantize(quantize(x))``, float32, shape ``x.shape[:-1]``
        (keys_values/kvcache/quantize/pytorch.py:530-548); x (B, Hkv, n, D). Uses scratch buffers, not
        the cache."""
        _lib.require_gpu(x)
        if x.ndim != 4 or x.shape[1] != self.shape[1] or x.shape[3] != self.shape[3]:
            raise ValueError(f"x.shape = {tuple(x.shape)}, must be (batch, {self.shape[1]}, n, {self.shape[3]})")
        xs = self._kernel_view(x.to(self.source_dtype))
        b, hkv, n, d = xs.shape
        dev = xs.device
        lib = _lib.load()
        first = b if self.blocks_over_heads else b * hkv
        with torch.cuda.device(dev):
            st = _lib.stream_ptr(dev)
            codes = torch.empty((first, n, self.blocksize * self.num_bits // 8), dtype=torch.uint8, device=dev)
            sc = torch.empty((first, n), dtype=torch.float32, device=dev)
            zp = torch.empty((first, n), dtype=torch.int32, device=dev)
            back = torch.empty((b, hkv, n, d), dtype=self.source_dtype, device=dev)
            _lib.check(lib.kvx_quantize_blocks(ctypes.byref(self._block_args(xs, 0, codes, sc, zp)), st))
            _lib.check(lib.kvx_dequantize_blocks(ctypes.byref(self._block_args(back, 0, codes, sc, zp)), st))
        return torch.linalg.vector_norm(xs - back, dim=-1, dtype=torch.float32)  # difference in the source dtype, as the reference


class RowQuantizer8(RowQuantizer):
    """8-bit codes, one block per (token, head) row: the store the attention kernels read directly."""

    def __init__(self, shape, source_dtype: torch.dtype = torch.bfloat16, num_bits: int = 8, blocks_over_heads: bool = False,
                 allocate_buffers: bool = False, device: Optional[torch.device] = None):
        if num_bits != 8:
            raise NotImplementedError(f"num_bits = {num_bits}: RowQuantizer8 is the 8-bit store; use RowQuantizer")
        if blocks_over_heads:
            raise NotImplementedError("blocks_over_heads=True: use RowQuantizer")
        super().__init__(shape, source_dtype, 8, False, allocate_buffers, device)
