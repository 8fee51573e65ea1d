"""
CPU oracle for the attention-with-score-sums + KV-cache path.  TEST INFRASTRUCTURE ONLY.

This module restates, op for op, the eager (CPU-capable) path of awslabs/keys_values so that the
HIP kernels have something to be compared with.  Only tests, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it; the library never does.

Every function cites the reference lines it follows (paths relative to the reference root).
How each function is pinned (tests/test_oracle.py):

* ``sdpa_in_blocks`` / ``sdpa_noblock`` / ``lse2``: brute force in float64 (``weights_bruteforce_f64``,
  written as explicit loops from the formula in test/attention/test_attn_weights.py:51-101), the
  library routine ``torch.nn.functional.scaled_dot_product_attention(is_causal=True)`` on the
  square case, closed forms (uniform keys, q_len == 1), the invariants of
  test/attention/test_flashinfer_wrapper.py:420-454 (W >= 0, rows sum to q_len), GQA == mean of the
  per-head result (test/attention/test_attention.py:78-166), blocked == unblocked
  (test/attention/test_attention.py:706-797), reorder == position mask
  (test/attention/test_sdpa_wrapper.py:55-153), and the independent scalar C restatement.
* ``quantize_rows`` / ``dequantize_rows`` (8 and 4 bits), ``compress4`` / ``uncompress4``,
  ``quantize_store`` / ``dequantize_store``: the known-answer round trip of
  test/kvcache/test_quantization.py:647-766 (integers with both extremes in every block, rows and
  blocks over heads), hand-computed vectors and packed bytes, and bit-equality with the scalar C
  restatement (IEEE float32 primitives only).
* ``h2o_update_select`` / ``cache_write`` / ``H2OCacheOracle``: brute-force python loops on small caches
  and the bookkeeping checks of test/kvcache/test_h2o.py:109-137,227-343; the normalised selection
  (scores divided by residency, keys_values/kvcache/h2o.py:183-196) by per-slot loops in numpy float32
  on data that tells the clamp at prefill_length - 1 and the already advanced input_pos from their
  off-by-one neighbours, and at cache level by a per-token model (tests/test_policy_oracle.py).
* Tie order of ``torch.argsort`` / ``torch.topk(sorted=False)`` is implementation-defined in the
  reference (keys_values/kvcache/attn_weights.py:773-783): parity unpinned for ties; this oracle and
  the kernels both break ties towards the lower slot and tests compare sets away from ties.
"""

import math
from typing import Optional, Tuple

import numpy as np
import torch

F32_MIN = torch.finfo(torch.float32).min
F32_EPS = torch.finfo(torch.float32).eps  # 1.1920929e-07, keys_values/kvcache/quantize/pytorch.py:76
TMP_LIMIT_GB_DEFAULT = 3.0  # keys_values/attention/attention_utils.py:304-360 (temp array limit)


# --------------------------------------------------------------------------------------------
# Attention
# --------------------------------------------------------------------------------------------


def _scores(query: torch.Tensor, key: torch.Tensor, scale: float) -> torch.Tensor:
    """keys_values/attention/attention_utils.py:69-122: the scale is folded into the smaller
    operand before the (grouped) matmul. query (B,Hq,q,D) fp32, key (B,Hkv,T,D) fp32."""
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    G = Hq // Hkv
    kt = key.mT
    if scale == 1.0:
        a = query
    elif query.numel() <= key.numel():
        a = query * scale
    else:
        kt = kt * scale
        a = query
    if G == 1:
        return torch.matmul(a, kt)
    s = torch.matmul(a.view(B, Hkv, G, q_len, D), kt.unsqueeze(2))
    return s.view(B, Hq, q_len, T)


def _masked(query_pos0: int, num: int, token_positions: torch.Tensor, Hq: int) -> torch.Tensor:
    """keys_values/attention/attention_utils.py:205-247: True where the pair is MASKED, i.e.
    query position < token position. token_positions (B,Hkv,T) -> (B,Hq,num,T)."""
    B, Hkv, T = token_positions.shape
    G = Hq // Hkv
    tp = token_positions.unsqueeze(2).expand(-1, -1, G, -1).reshape(B, Hq, 1, T)
    qpos = torch.arange(query_pos0, query_pos0 + num, dtype=token_positions.dtype).view(1, 1, -1, 1)
    return qpos < tp


def _tmp_len(B: int, Hq: int, q_len: int, T: int, limit_gb: float) -> int:
    """keys_values/attention/attention_utils.py:316-360: number of query rows per slice so that
    the fp32 score array (B,Hq,tmp_len,T) stays under the limit."""
    per_row = B * Hq * T * 4
    return max(1, min(q_len, int(limit_gb * (2**30)) // per_row))


def sdpa_in_blocks(
    query: torch.Tensor,
    key: torch.Tensor,
    value: torch.Tensor,
    scale_factor: float,
    input_pos: int,
    token_positions: Optional[torch.Tensor],
    return_attn_weights: bool = True,
    tmp_array_limit_gb: float = TMP_LIMIT_GB_DEFAULT,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """keys_values/attention/base.py:660-742 (scaled_dot_product_attention_in_blocks) with
    keys_values/attention/attention_utils.py:383-443 (sdpa_attention_weights).

    query (B,Hq,q,D), key/value (B,Hkv,T,D) in fp32/bf16/fp16; token_positions (B,Hkv,T) int or None.
    Returns O (B,Hq,q,D) in query.dtype and W (B,Hkv,T) fp32 (sum over queries, mean over group)."""
    dtype = query.dtype
    key32 = key.to(torch.float32)
    value32 = value.to(torch.float32)
    B, Hq, q_len, D = query.shape
    Hkv, T = key32.shape[1], key32.shape[2]
    G = Hq // Hkv
    if token_positions is None:  # attention_utils.py:425-432
        token_positions = torch.arange(T, dtype=torch.int64).view(1, 1, T).expand(B, Hkv, T)
    tmp_len = _tmp_len(B, Hq, q_len, T, tmp_array_limit_gb)
    parts = []
    weights = 0
    for start in range(0, q_len, tmp_len):
        end = min(start + tmp_len, q_len)
        sz = end - start
        s = _scores(query[:, :, start:end, :].to(torch.float32), key32, scale_factor)
        s[_masked(input_pos + start, sz, token_positions, Hq)] = F32_MIN  # attention_utils.py:441
        p = s.softmax(dim=-1)  # attention_utils.py:443
        if return_attn_weights:
            src = p if G == 1 else torch.mean(p.view(B, Hkv, G, sz, T), dim=2)  # base.py:707-724
            weights = src.sum(dim=2) + weights  # base.py:725
        if G == 1:
            o = torch.matmul(p, value32)
        else:
            o = torch.matmul(p.view(B, Hkv, G, sz, T), value32.unsqueeze(2)).view(B, Hq, sz, D)
        parts.append(o.to(dtype))  # base.py:730-735
    out = torch.cat(parts, dim=2)
    return out, (weights if return_attn_weights else None)


def sdpa_noblock(query, key, value, scale_factor, input_pos, token_positions, return_attn_weights=True):
    """keys_values/attention/base.py:620-645 (eager path, use_blocking=False) with the additive
    mask built as in keys_values/kvcache/test_utils.py:171-201: scores*scale, + (-inf where masked),
    softmax, sum over queries, mean over the group."""
    dtype = query.dtype
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    G = Hq // Hkv
    if token_positions is None:
        token_positions = torch.arange(T, dtype=torch.int64).view(1, 1, T).expand(B, Hkv, T)
    s = _scores(query.to(torch.float32), key.to(torch.float32), 1.0) * scale_factor
    mask = torch.zeros_like(s)
    mask[_masked(input_pos, q_len, token_positions, Hq)] = float("-inf")
    p = torch.softmax(s + mask, dim=-1)
    v32 = value.to(torch.float32)
    o = torch.matmul(p.view(B, Hkv, G, q_len, T), v32.unsqueeze(2)).view(B, Hq, q_len, D).to(dtype)
    w = None
    if return_attn_weights:
        w = p.sum(dim=2)
        if G > 1:
            w = w.view(B, Hkv, G, T).mean(dim=2)
    return o, w


def lse2(query, key, scale_factor, input_pos, token_positions) -> torch.Tensor:
    """Base-2 log-sum-exp of the masked, scaled scores, layout (B, q, Hq):
    keys_values/csrc/kernels/sdpa_prefill.cu:509-512, test/attention/test_flashinfer_wrapper.py:1175-1200
    (torch.logsumexp / ln 2)."""
    B, Hq, q_len, D = query.shape
    Hkv, T = key.shape[1], key.shape[2]
    if token_positions is None:
        token_positions = torch.arange(T, dtype=torch.int64).view(1, 1, T).expand(B, Hkv, T)
    s = _scores(query.to(torch.float32), key.to(torch.float32), 1.0) * scale_factor
    s = s.masked_fill(_masked(input_pos, q_len, token_positions, Hq), float("-inf"))
    return (torch.logsumexp(s, dim=-1) / math.log(2.0)).permute(0, 2, 1).contiguous()


def weights_bruteforce_f64(query, key, value, scale, input_pos, token_positions):
    """Explicit float64 loops over (b, head, query, key): the formula of
    test/attention/test_attn_weights.py:51-101 written without any library softmax/matmul.
    Small shapes only. Returns (O (B,Hq,q,D), W (B,Hkv,T), LSE2 (B,q,Hq)) as float64 numpy."""
    q = query.double().numpy()
    k = key.double().numpy()
    v = value.double().numpy()
    B, Hq, q_len, D = q.shape
    Hkv, T = k.shape[1], k.shape[2]
    G = Hq // Hkv
    tp = np.broadcast_to(np.arange(T), (B, Hkv, T)) if token_positions is None else token_positions.numpy()
    O = np.zeros((B, Hq, q_len, D))
    W = np.zeros((B, Hkv, T))
    L = np.zeros((B, q_len, Hq))
    for b in range(B):
        for h in range(Hq):
            g = h // G  # attention_utils.py:111-122: head h reads KV head h // G
            for i in range(q_len):
                logits = np.full(T, -np.inf)
                for t in range(T):
                    if tp[b, g, t] <= input_pos + i:
                        logits[t] = scale * float(np.dot(q[b, h, i], k[b, g, t]))
                m = logits.max()
                e = np.exp(logits - m)
                z = e.sum()
                p = e / z
                O[b, h, i] = p @ v[b, g]
                W[b, g] += p / G
                L[b, i, h] = (m + math.log(z)) / math.log(2.0)
    return O, W, L


def reorder_key_value(key, value, token_positions):
    """keys_values/attention/sdpa_wrapper.py:352-369: sort the slots of every (b, h) row by token
    position so that a right-aligned causal mask applies. Returns sorted K, V and the sort index."""
    idx = torch.argsort(token_positions.to(torch.int64), dim=-1)
    gi = idx.unsqueeze(-1).expand(-1, -1, -1, key.shape[-1])
    return key.gather(2, gi), value.gather(2, gi), idx


# --------------------------------------------------------------------------------------------
# 8-bit affine row quantiser
# --------------------------------------------------------------------------------------------


def quantize_rows(x: torch.Tensor, num_bits: int = 8) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """keys_values/kvcache/quantize/pytorch.py:312-355 (_quantize), :100-116 (_calculate_qparams),
    :120-139 (quantize_per_channel), one block per row; quant_max = 2**num_bits - 1 (:191-196).
    x (..., D) any float dtype. Returns codes uint8 (..., D) (not packed), scale fp32 (...), zp int32 (...)."""
    shape = x.shape
    qmax = 2**num_bits - 1
    v = x.to(torch.float32).reshape(-1, shape[-1])  # :333
    mn, mx = torch.aminmax(v, dim=1)  # :90
    scale = torch.clamp((mx - mn) / float(qmax - 0), min=F32_EPS)  # :111-114
    zp = 0 - torch.round(mn / scale).to(torch.int32)  # :115
    res = torch.clamp(torch.round(v * (1.0 / scale.view(-1, 1))) + zp.view(-1, 1), 0, qmax)  # :134-138
    return res.to(torch.uint8).reshape(shape), scale.reshape(shape[:-1]), zp.reshape(shape[:-1])


def dequantize_rows(codes: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor, dtype=torch.bfloat16):
    """keys_values/kvcache/quantize/pytorch.py:143-154 (dequantize_per_channel), :467-478:
    (codes - zp) * scale in the promoted types (uint8 - int32 -> int32, * fp32 -> fp32), then the
    source dtype."""
    res = (codes - zp.unsqueeze(-1)) * scale.unsqueeze(-1)
    return res.to(torch.float32).to(dtype)


def compress4(codes: torch.Tensor) -> torch.Tensor:
    """keys_values/kvcache/quantize/pytorch.py:384-393: byte j = code[j] << 4 | code[j + n/2]."""
    half = codes.shape[-1] // 2
    return torch.bitwise_or(torch.bitwise_left_shift(codes[..., :half], 4), codes[..., half:])


def uncompress4(packed: torch.Tensor) -> torch.Tensor:
    """keys_values/kvcache/quantize/pytorch.py:457-465."""
    return torch.cat((torch.bitwise_right_shift(packed, 4), torch.bitwise_and(packed, 15)), dim=-1)


def quantize_store(values: torch.Tensor, num_bits: int = 8, blocks_over_heads: bool = False):
    """What TorchBasicQuantizer.quantize leaves in its buffers for values (B, Hkv, n, D)
    (keys_values/kvcache/quantize/pytorch.py:235-245,312-355): quant_buffer (first, n, final) uint8 with
    first = B*Hkv, final = D[/2], or first = B, final = Hkv*D[/2] when the blocks run over the heads
    (values transposed to (B, n, Hkv, D) first, :335-337); quant_scales / quant_zero_points (first, n)."""
    B, Hkv, n, D = values.shape
    v = values.transpose(1, 2).reshape(B, n, Hkv * D) if blocks_over_heads else values.reshape(B * Hkv, n, D)
    codes, scale, zp = quantize_rows(v, num_bits)
    if num_bits == 4:
        codes = compress4(codes)
    return codes, scale, zp


def dequantize_store(buffer, scale, zp, shape, num_bits: int = 8, blocks_over_heads: bool = False, dtype=torch.bfloat16):
    """Inverse of quantize_store, to (B, Hkv, n, D) (keys_values/kvcache/quantize/pytorch.py:411-478)."""
    B, Hkv, n, D = shape
    codes = uncompress4(buffer) if num_bits == 4 else buffer
    out = dequantize_rows(codes, scale, zp, dtype)
    if blocks_over_heads:
        return out.reshape(B, n, Hkv, D).transpose(1, 2)
    return out.reshape(B, Hkv, n, D)


def quantization_error(x: torch.Tensor, num_bits: int = 8) -> torch.Tensor:
    """keys_values/kvcache/quantize/pytorch.py:530-548: per-row L2 norm of x - dequant(quant(x)); the
    dequantised rows and the difference are in the source dtype, the norm accumulates in float32."""
    c, s, z = quantize_rows(x, num_bits)
    return torch.linalg.vector_norm(x - dequantize_rows(c, s, z, x.dtype), dim=-1, dtype=torch.float32)


# --------------------------------------------------------------------------------------------
# Cache write and H2O bookkeeping
# --------------------------------------------------------------------------------------------


def cache_write(k_cache, v_cache, token_pos, scores, index, key, value, input_pos):
    """In place. keys_values/kvcache/attn_weights.py:305-316 (token_pos scatter), :679-681 (scores
    scatter of 0), keys_values/kvcache/buffers.py:498-519 (K/V scatter_ along the slot axis).
    index (B,Hkv,num) int64; key/value (B,Hkv,num,D)."""
    B, Hkv, num = index.shape
    D = key.shape[-1]
    new_tp = torch.arange(input_pos, input_pos + num, dtype=token_pos.dtype).view(1, 1, -1).expand(B, Hkv, num)
    token_pos[:B].scatter_(-1, index, new_tp)
    gi = index.unsqueeze(-1).expand(-1, -1, -1, D)
    k_cache[:B].scatter_(-2, gi, key.to(k_cache.dtype))
    v_cache[:B].scatter_(-2, gi, value.to(v_cache.dtype))
    if scores is not None:
        scores[:B].scatter_(-1, index, 0.0)


def select_smallest(values: torch.Tensor, k: int) -> torch.Tensor:
    """First k entries of a stable ascending argsort along the last axis: what
    keys_values/kvcache/attn_weights.py:773-774 consumes (`argsort` then `[:, :, :num]`), with ties
    resolved to the lower slot."""
    return torch.argsort(values, dim=-1, stable=True)[..., :k]


def h2o_update_select(scores, w, kv_len, limit, k, normalize=False, token_pos=None, input_pos=0, prefill_len=0):
    """In place on scores. keys_values/kvcache/h2o.py:175-196 and
    keys_values/kvcache/attn_weights.py:771-783. scores (B,Hkv,L) fp32, w (B,Hkv,kv_len) fp32 or None.
    Returns next_index (B,Hkv,k) int64."""
    B = scores.shape[0] if w is None else w.shape[0]
    if w is not None:
        scores[:B, :, :kv_len] += w
    s = scores[:B, :, :limit]
    if normalize:  # h2o.py:183-196; input_pos has already been advanced
        tp = token_pos[:B, :, :limit].maximum(torch.full((1, 1, 1), prefill_len - 1, dtype=token_pos.dtype))
        s = s / (input_pos - tp).to(torch.float32)
    return select_smallest(s, k)


class H2OCacheOracle:
    """One layer's H2O cache, restating the step order of DefaultKVCache.forward
    (keys_values/kvcache/base.py:554-595): evict-write -> attend -> score -> select, for a full
    cache without grace period (keys_values/kvcache/attn_weights.py:510-635,721-783;
    keys_values/kvcache/h2o.py:146-199). prefill() follows :817-869 (no weights on the first chunk)
    and the one-off initial rule follows :536-550."""

    KEEP_INITIAL_FRACTION = 0.05  # attn_weights.py:322

    def __init__(self, B, Hq, Hkv, L, D, dtype=torch.float32, max_chunk_size=None):
        self.B, self.Hq, self.Hkv, self.L, self.D = B, Hq, Hkv, L, D
        self.k = torch.zeros(B, Hkv, L, D, dtype=dtype)
        self.v = torch.zeros(B, Hkv, L, D, dtype=dtype)
        self.token_pos = torch.zeros(B, Hkv, L, dtype=torch.int32)
        self.scores = torch.zeros(B, Hkv, L, dtype=torch.float32)
        self.max_chunk_size = None if (max_chunk_size is None or max_chunk_size > L // 2) else max_chunk_size  # :458-462
        self.input_pos = 0
        self.current_length = 0
        self.next_index = None
        self.use_initial_rule = False
        self.scale = 1.0 / math.sqrt(D)

    def prefill(self, query, key, value, store_key=None, store_value=None):
        """The first chunk attends over key / value as given (keys_values/kvcache/base.py:567-571);
        store_key / store_value are what the buffers hold afterwards when they differ (a quantised
        store holds the dequantised rows)."""
        n = key.shape[2]
        assert n <= self.L
        self.k[:, :, :n] = (key if store_key is None else store_key).to(self.k.dtype)
        self.v[:, :, :n] = (value if store_value is None else store_value).to(self.v.dtype)
        self.token_pos[:, :, :n] = torch.arange(n, dtype=torch.int32)
        self.scores.zero_()
        self.current_length = n
        self.input_pos = n
        self.use_initial_rule = n == self.L
        self.next_index = None
        o, _ = sdpa_in_blocks(query, key, value, self.scale, 0, None, return_attn_weights=False)
        return o

    def forward(self, query, key, value):
        num = key.shape[2]
        if self.current_length < self.L:  # free slots, attn_weights.py:1001-1016
            assert self.current_length + num <= self.L
            index = torch.arange(self.current_length, self.current_length + num).view(1, 1, -1).expand(self.B, self.Hkv, -1)
            self.current_length += num
        elif self.use_initial_rule:  # :536-550
            n0 = min(int(self.KEEP_INITIAL_FRACTION * self.L), self.L - num)
            index = torch.arange(n0, n0 + num).view(1, 1, -1).expand(self.B, self.Hkv, -1)
            self.use_initial_rule = False
        else:
            index = self.next_index[:, :, :num]
        index = index.contiguous().to(torch.int64)
        cache_write(self.k, self.v, self.token_pos, self.scores, index, key, value, self.input_pos)
        T = self.current_length
        o, w = sdpa_in_blocks(
            query, self.k[:, :, :T], self.v[:, :, :T], self.scale, self.input_pos, self.token_pos[:, :, :T].to(torch.int64)
        )
        self.input_pos += num
        if T == self.L:
            k = self.L if self.max_chunk_size is None else self.max_chunk_size
            self.next_index = h2o_update_select(self.scores, w, T, self.L, k)
        else:
            self.scores[:, :, :T] += w
        return o, w, index


# --------------------------------------------------------------------------------------------
# RoPE used to build the benchmark inputs (not part of the kernels)
# --------------------------------------------------------------------------------------------


def apply_rope(x: torch.Tensor, positions: torch.Tensor, theta: float = 1e6) -> torch.Tensor:
    """Half-split rotation y = x*cos + cat(-x2, x1)*sin (keys_values/fused/fused_rope.py:57-87,198-200).
    x (..., T, D); positions (..., T) broadcastable."""
    D = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    ang = positions.to(torch.float32).unsqueeze(-1) * inv
    cos = torch.cat((ang.cos(), ang.cos()), dim=-1)
    sin = torch.cat((ang.sin(), ang.sin()), dim=-1)
    x32 = x.to(torch.float32)
    x1, x2 = x32[..., : D // 2], x32[..., D // 2 :]
    return (x32 * cos + torch.cat((-x2, x1), dim=-1) * sin).to(x.dtype)
