"""
``RowQuantizer8``: the 8-bit case of ``TorchBasicQuantizer``
(keys_values/kvcache/quantize/pytorch.py:157-564) on the HIP kernels, one quantisation block per
(token, head) row. Same buffer names, shapes and dtypes (``quant_buffer`` uint8 ``(B*Hkv, L, D)``,
``quant_scales`` float32 ``(B*Hkv, L)``, ``quant_zero_points`` int32 ``(B*Hkv, L)``, :281-295), same
methods with the same meaning (``allocate_buffers``, ``deallocate``, ``quantize``, ``dequantize``,
``quantization_error``; keys_values/kvcache/quantize/quantization.py:102-236). Codes, scales and
zero points are bit-identical to the reference's for every row whose zero point fits int32.

Not covered (raises): 4-bit packing and ``blocks_over_heads=True`` (:235-245, :384-393).
"""
from typing import Optional, Tuple

import torch

from .. import _lib


class RowQuantizer8:
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
        if num_bits != 8:
            raise NotImplementedError(f"num_bits = {num_bits}: only the 8-bit store is implemented")
        if blocks_over_heads:
            raise NotImplementedError("blocks_over_heads=True is not implemented")
        if source_dtype != torch.bfloat16:
            raise NotImplementedError(f"source_dtype = {source_dtype}: the kernels take bfloat16 rows")
        if shape[3] not in (64, 128):
            raise NotImplementedError(f"head_size = {shape[3]} not in (64, 128)")
        self.shape = tuple(shape)
        self.source_dtype = source_dtype
        self.blocks_over_heads = False
        self.max_batch_size, self.n_query_groups = shape[0], shape[1]
        self.blocksize = shape[3]
        self.quant_buffer = None
        self.quant_scales = None
        self.quant_zero_points = None
        self._batch_size = None
        if allocate_buffers:
            self.allocate_buffers(shape[0], device)

    # -- buffers (keys_values/kvcache/quantize/pytorch.py:253-310) ---------------------------------

    @property
    def device(self) -> Optional[torch.device]:
        return self.quant_buffer.device if self.quant_buffer is not None else None

    @property
    def batch_size(self) -> Optional[int]:
        return self._batch_size

    @property
    def buffers_are_allocated(self) -> bool:
        return self.quant_buffer is not None

    def allocate_buffers(self, batch_size: int, device: Optional[torch.device] = None):
        if not (0 < batch_size <= self.max_batch_size):
            raise ValueError(f"batch_size = {batch_size} must be in (0, {self.max_batch_size}]")
        if device is None:
            device = self.device if self.buffers_are_allocated else torch.device("cuda", torch.cuda.current_device())
        device = torch.device(device)
        if device.type != "cuda":
            raise RuntimeError(f"RowQuantizer8 buffers live on a ROCm device, not on {device}: there is no CPU path")
        if (not self.buffers_are_allocated) or batch_size > self.shape[0] or device != self.device:
            self.shape = (batch_size,) + self.shape[1:]
            _, hkv, length, d = self.shape
            self.quant_buffer = torch.empty((batch_size * hkv, length, d), dtype=torch.uint8, device=device)
            self.quant_scales = torch.zeros((batch_size * hkv, length), dtype=torch.float32, device=device)
            self.quant_zero_points = torch.zeros((batch_size * hkv, length), dtype=torch.int32, device=device)
        self._batch_size = batch_size

    def deallocate(self):
        self.quant_buffer = None
        self.quant_scales = None
        self.quant_zero_points = None
        self._batch_size = None

    def _views(self):
        """(B, Hkv, L, D) codes and (B, Hkv, L) state views of the flat buffers."""
        b, hkv, length, d = self._batch_size, self.shape[1], self.shape[2], self.shape[3]
        n = b * hkv
        return (
            self.quant_buffer[:n].view(b, hkv, length, d),
            self.quant_scales[:n].view(b, hkv, length),
            self.quant_zero_points[:n].view(b, hkv, length),
        )

    # -- quantise / dequantise -----------------------------------------------------------------------

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
            if start == 0 and end == length and values.is_contiguous():
                rows = b * hkv * length
                _lib.check(lib.kvx_quantize_rows(values.data_ptr(), d, rows, d, self.quant_buffer.data_ptr(),
                                                  self.quant_scales.data_ptr(), self.quant_zero_points.data_ptr(), st))
                return
            # one launch per (b, h) row block: rows inside it are `num` consecutive slots
            for i in range(b * hkv):
                src = values[i // hkv, i % hkv]
                if src.stride(-1) != 1 or src.stride(0) % 8 != 0 or src.data_ptr() % 16 != 0:
                    src = src.contiguous()
                _lib.check(lib.kvx_quantize_rows(
                    src.data_ptr(), src.stride(0), num, d,
                    self.quant_buffer[i, start:end].data_ptr(), self.quant_scales[i, start:end].data_ptr(),
                    self.quant_zero_points[i, start:end].data_ptr(), st))

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
            st = _lib.stream_ptr(dev)
            for i in range(b * hkv):
                _lib.check(lib.kvx_dequantize_rows(
                    self.quant_buffer[i, start:end].data_ptr(), self.quant_scales[i, start:end].data_ptr(),
                    self.quant_zero_points[i, start:end].data_ptr(), num, d, out[i // hkv, i % hkv].data_ptr(), d, st))
        return out

    def quantization_error(self, x: torch.Tensor) -> torch.Tensor:
        """Per-row L2 norm of ``x - dequantize(quantize(x))``, float32, shape ``x.shape[:-1]``
        (keys_values/kvcache/quantize/pytorch.py:530-548). Uses scratch buffers, not the cache."""
        _lib.require_gpu(x)
        d = x.shape[-1]
        xs = x.to(self.source_dtype).reshape(-1, d).contiguous()
        rows = xs.shape[0]
        dev = xs.device
        lib = _lib.load()
        with torch.cuda.device(dev):
            st = _lib.stream_ptr(dev)
            codes = torch.empty((rows, d), dtype=torch.uint8, device=dev)
            sc = torch.empty(rows, dtype=torch.float32, device=dev)
            zp = torch.empty(rows, dtype=torch.int32, device=dev)
            back = torch.empty((rows, d), dtype=self.source_dtype, device=dev)
            _lib.check(lib.kvx_quantize_rows(xs.data_ptr(), d, rows, d, codes.data_ptr(), sc.data_ptr(), zp.data_ptr(), st))
            _lib.check(lib.kvx_dequantize_rows(codes.data_ptr(), sc.data_ptr(), zp.data_ptr(), rows, d, back.data_ptr(), d, st))
        err = torch.linalg.vector_norm(xs - back, dim=-1, dtype=torch.float32)  # difference in the source dtype, as the reference
        return err.reshape(x.shape[:-1])
