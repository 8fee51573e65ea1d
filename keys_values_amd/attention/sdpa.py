"""
``HipSDPA``: the drop-in for ``FlashInferSDPA`` (keys_values/attention/flashinfer_wrapper.py:322-682).

``scaled_dot_product_attention`` keeps the reference's signature, shapes, routing and errors
(:367-510). What is gone is the data movement the reference needs around its kernels: no sort and
gather of the cache by ``token_positions`` (keys_values/attention/sdpa_wrapper.py:352-369) and no
un-permuting of the weights (:492-494), because the kernels apply the position mask themselves
(``token_positions[b,h,k] <= input_pos + i``, keys_values/attention/attention_utils.py:238-247), and
no ``transpose(1, 2).contiguous()`` of Q, K, V (:590-592), because they take strides.
"""
import math
from typing import Optional, Tuple

import torch

from . import ops

_PAD_TO = ops.ALLOWED_HEAD_SIZES


def can_do_hip_sdpa(head_size: int, dtype: torch.dtype, return_attn_weights: bool = False) -> bool:
    """Gate with the meaning of ``can_do_flashinfer`` (keys_values/attention/flashinfer_wrapper.py:311-319)."""
    return dtype in ops.ALLOWED_DTYPES and 0 < head_size <= _PAD_TO[-1] and ops.is_available()


def _pad_head_size(query, key, value):
    """Zero-pad the head dimension up to the next supported size, as ``pad_head_size`` does
    (keys_values/attention/flashinfer_wrapper.py:279-308); zeros change neither scores nor outputs."""
    head_size = query.shape[-1]
    target = next((s for s in _PAD_TO if head_size <= s), None)
    if target is None:
        raise NotImplementedError(f"head_size <= {_PAD_TO[-1]} needed, but is {head_size}")
    diff = target - head_size
    if diff == 0:
        return query, key, value, None
    pad = lambda t: torch.nn.functional.pad(t, (0, diff))  # noqa: E731
    return pad(query), pad(key), pad(value), diff


def sdpa_check_args(query, key, value, packed4: bool = False):
    """keys_values/attention/sdpa_wrapper.py:24-47. ``packed4``: key / value are rows of the 4-bit store, two
    codes per byte, so their last axis is half the head size."""
    if query.ndim != 4 or key.ndim != 4 or value.ndim != 4:
        raise ValueError("query, key, value must be 4D tensors")
    if key.shape != value.shape:
        raise ValueError("key, value must have same shape")
    batch_size, n_head, q_len, head_size = query.shape
    if key.shape[0] != batch_size or key.shape[-1] != (head_size // 2 if packed4 else head_size):
        raise ValueError(f"key.shape = {key.shape}, must be ({batch_size}, _, _, {head_size})")
    _, n_query_groups, kv_len, _ = key.shape
    if not (0 < q_len <= kv_len):
        raise ValueError(f"Must have 0 < q_len = {q_len} <= kv_len = {kv_len}. Don't use this for prefill")
    if n_query_groups <= 0 or n_head % n_query_groups != 0 or n_head < n_query_groups:
        raise ValueError(
            f"n_head = {n_head}, n_query_groups = {n_query_groups}: n_head must be positive multiple of n_query_groups"
        )
    return batch_size, n_head, n_query_groups, q_len, kv_len, head_size


class HipSDPA:
    """Same call surface as ``FlashInferSDPA``; ``available`` replaces its constructor-time probe
    (keys_values/attention/flashinfer_wrapper.py:331-365)."""

    def __init__(self):
        self.available = ops.is_available()

    def scaled_dot_product_attention(
        self,
        query: torch.Tensor,
        key: torch.Tensor,
        value: torch.Tensor,
        scale_factor: Optional[float],
        input_pos: int,
        token_positions: Optional[torch.Tensor],
        return_attn_weights: bool = False,
        sort_if_3d: bool = True,
        output_transposed: bool = False,
        quant: Optional[ops.QuantState] = None,
    ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """query (B, n_head, q_len, hs); key/value (B, n_query_groups, kv_len, hs), possibly strided
        views of a larger cache; ``token_positions`` (B, n_query_groups, kv_len) or None (= arange).
        Returns ``(attn_outputs, attn_weights)``: outputs (B, n_head, q_len, hs), or
        (B, q_len, n_head, hs) if ``output_transposed``; weights fp32 (B, n_query_groups, kv_len) or None.
        ``sort_if_3d`` is accepted for compatibility and has no effect (nothing is sorted).
        ``quant`` (not in the reference) marks key/value as uint8 codes with their per-row state."""
        if not isinstance(input_pos, int):
            raise ValueError("input_pos must be int scalar")
        if input_pos <= 0:
            raise ValueError("input_pos must be positive. Don't use for square prefill")
        packed4 = quant is not None and key.ndim == 4 and query.ndim == 4 and key.shape[-1] * 2 == query.shape[-1]
        batch_size, n_head, n_query_groups, q_len, kv_len, head_size = sdpa_check_args(query, key, value, packed4)
        if token_positions is not None and token_positions.shape != key.shape[:-1]:
            raise ValueError(f"token_positions.shape = {token_positions.shape}, key.shape = {key.shape}: Not compatible")
        if scale_factor is None:
            scale_factor = 1.0 / math.sqrt(head_size)
        if query.dtype not in ops.ALLOWED_DTYPES or head_size > _PAD_TO[-1]:
            raise NotImplementedError(
                "HipSDPA needs these conditions:\n"
                f"- head_size <= {_PAD_TO[-1]}, but is {head_size}\n"
                f"- query.dtype in (torch.bfloat16, torch.float16), but is {query.dtype}"
            )
        use_decode_kernel = q_len == 1
        if use_decode_kernel and kv_len == 1:
            raise NotImplementedError("Don't use for q_len=1, kv_len=1")
        if quant is None:
            query, key, value, head_size_diff = _pad_head_size(query, key, value)
        else:
            head_size_diff = None
            if head_size not in ops.QUANTIZED_HEAD_SIZES:
                raise NotImplementedError(f"quantised cache needs head_size in {ops.QUANTIZED_HEAD_SIZES}")

        if use_decode_kernel:
            # the single new token is the newest: it sees every slot, positions are not needed
            # (keys_values/attention/flashinfer_wrapper.py:471-481)
            out, attn_weights, _ = ops.decode_core(query, key, value, scale_factor, return_attn_weights, quant=quant)
            attn_outputs = out.unsqueeze(1) if output_transposed else out.unsqueeze(2)
        else:
            attn_outputs, attn_weights, _ = ops.prefill_core(
                query, key, value, scale_factor, input_pos, token_positions, return_attn_weights,
                return_lse=False, output_transposed=output_transposed, quant=quant,
            )
        if head_size_diff is not None:
            attn_outputs = attn_outputs[:, :, :, :head_size]
        return attn_outputs, attn_weights


class HipMultiHeadSelfAttention:
    """The call surface of ``MultiHeadSelfAttention.__call__`` (keys_values/attention/base.py:287-380) for the
    configurations the HIP kernels serve (no sliding window, no logit soft-capping): the cache passes the
    queries and a ``KeysAndValues`` holder and gets ``(attn_outputs (B, q_len, n_head * hs), attn_weights)``.
    ``input_pos`` 0 / None is the causal first chunk (no weights, keys_values/kvcache/base.py:567-581). A holder
    of a quantised store (``key_codes`` / ``value_codes`` / ``quant``) is read in place by the kernels."""

    def __init__(self, scale_factor: Optional[float] = None):
        self.scale_factor = scale_factor
        self._sdpa = get_hip_sdpa()

    def __call__(self, query: torch.Tensor, k_and_v, block_idx: int = 0, input_pos: Optional[int] = None,
                 return_attn_weights: bool = False, token_positions: Optional[torch.Tensor] = None):
        is_causal = input_pos is None or input_pos == 0
        if not is_causal and token_positions is None:
            raise ValueError("token_positions must be given if input_pos > 0")
        quant = getattr(k_and_v, "quant", None)
        if quant is not None:
            key, value = k_and_v.key_codes, k_and_v.value_codes
        else:
            key, value = k_and_v.keys(), k_and_v.values()
        batch_size, _, q_len, head_size = query.shape
        scale = self.scale_factor if self.scale_factor is not None else 1.0 / math.sqrt(head_size)
        if is_causal:
            if return_attn_weights:
                raise ValueError("attention weights are not returned for the first chunk (input_pos = 0)")
            if key.shape[2] != q_len:
                raise ValueError(f"first chunk: kv_len = {key.shape[2]} must equal q_len = {q_len}")
            if quant is None:
                query, key, value, diff = _pad_head_size(query, key, value)
            else:
                diff = None
            out, _, _ = ops.prefill_core(query, key, value, scale, 0, None, return_weights=False, output_transposed=True, quant=quant)
            if diff is not None:
                out = out[..., :head_size]
            return out.reshape(batch_size, q_len, -1), None
        out, w = self._sdpa.scaled_dot_product_attention(query, key, value, scale, input_pos, token_positions, return_attn_weights,
                                                         output_transposed=True, quant=quant)
        return out.reshape(batch_size, q_len, -1), w


_hip_sdpa = None


def get_hip_sdpa() -> Optional[HipSDPA]:
    """Lazy singleton like ``_get_flashinfer_sdpa`` (keys_values/attention/base.py:115-126)."""
    global _hip_sdpa
    if _hip_sdpa is None:
        _hip_sdpa = HipSDPA()
    return _hip_sdpa
