"""
CPU oracle for the eviction-policy variants of the H2O cache.  TEST INFRASTRUCTURE ONLY.

Restates, tensor op for tensor op, what awslabs/keys_values does for a cache with a grace period,
normalised scores, V-norm weighted instantaneous scores and the Q-Hitter combination with the
quantisation error.  Only tests may import it; the library never does.

Reference lines (paths relative to the reference root):
  grace period ring         keys_values/kvcache/attn_weights.py:267-303 (token positions),
                            :565-606 (fused copy + write), :636-681 (score buffers), :861-863
  wrap-around positions     keys_values/kvcache/buffers.py:80-132
  scores, normalisation     keys_values/kvcache/h2o.py:146-199
  V-norm weighting          keys_values/kvcache/h2o.py:266-341
  Q-Hitter                  keys_values/kvcache/qh2o.py:130-210
  replay log                keys_values/kvcache/attn_weights.py:43-204

How it is pinned (tests/test_policy_oracle.py):
* grace period: an independent model that keeps python objects per slot (no index arithmetic shared
  with this file), the invariants asserted by test/kvcache/test_h2o.py:49-106, and equality with
  ``H2OCacheOracle`` when the grace period is 0;
* V-norm weighting: rows of V with equal norms reduce it to plain H2O (the weights of one step sum to
  the number of queries), the increments sum to the number of queries, and the brute-force
  recomputation of test/kvcache/test_h2o.py:109-225 (scores from full attention over all tokens);
* Q-Hitter: combination constant 1 selects what plain H2O selects, constant 0 selects the rows with
  the largest quantisation error, the modified values stay in [(1 - c) / 2, 1], and the
  quantisation error is checked against explicit float loops.
* Replay log: the concatenation of its blocks is the concatenation of every step's slots, and
  ``extract_index`` is a slice of it, checked for every start and length on a small log.
* A quantised store here holds dequantise(quantise(row)) for every row written, and a row moved out
  of the ring is written once more (the reference reads it from the dequantised buffer and writes it
  back through the quantiser, keys_values/kvcache/quant_buffers.py:732-775): checked against the row
  quantiser applied by hand, twice for moved rows, once for all others.
"""

import math
from typing import Optional

import torch

from .kvx_oracle import dequantize_rows, quantization_error, quantize_rows, sdpa_in_blocks, select_smallest

KEEP_INITIAL_FRACTION = 0.05  # keys_values/kvcache/attn_weights.py:322


def positions_wrap_around(num: int, current: int, start: int, end: int) -> torch.Tensor:
    """keys_values/kvcache/buffers.py:118-132: `num` slots from `current`, wrapping from `end` to `start`."""
    assert start <= current < end and num <= end - start
    num1 = min(num, end - current)
    pos = torch.arange(current, current + num1)
    if num > num1:
        pos = torch.cat((pos, torch.arange(start, start + num - num1)))
    return pos


def min_max_normalize(x: torch.Tensor) -> torch.Tensor:
    """keys_values/kvcache/qh2o.py:196-210: over all dimensions but the first."""
    flat = x.reshape(x.size(0), -1)
    mn = flat.min(dim=-1, keepdim=True)[0]
    den = flat.max(dim=-1, keepdim=True)[0] - mn
    return ((flat - mn) / den).view(*x.shape)


def update_select(scores, w, kv_len, limit, k, normalize=False, token_pos=None, input_pos=0, prefill_len=0, v_norm=None,
                  q_errors=None, combination=0.5, q_len=1):
    """In place on scores (B, Hkv, L). keys_values/kvcache/attn_weights.py:766-783 with
    keys_values/kvcache/h2o.py:175-199 (accumulate, normalise), :297-314 (V-norm weighted increment)
    and keys_values/kvcache/qh2o.py:178-194 (combination with the quantisation errors).
    Returns (next_index (B, Hkv, k) int64, the values compared (B, Hkv, limit))."""
    B = w.shape[0]
    inst = w
    if v_norm is not None:
        sc = v_norm[:B, :, :kv_len] * w
        inst = (sc / sc.sum(dim=-1, keepdim=True)) * q_len
    scores[:B, :, :kv_len] += inst
    s = scores[:B, :, :limit]
    if normalize:  # input_pos has already been advanced
        tp = token_pos[:B, :, :limit].maximum(torch.full((1, 1, 1), prefill_len - 1, dtype=token_pos.dtype))
        s = s / (input_pos - tp).to(torch.float32)
    if q_errors is not None:
        c = combination
        s = c * min_max_normalize(s) + ((c - 1) / 2) * min_max_normalize(q_errors[:B, :, :limit]) + (1 - c)
    return select_smallest(s, k), s


class ReplayLogOracle:
    """keys_values/kvcache/attn_weights.py:43-204: slot positions of the tokens from cache_length on, in
    blocks of `blocksize` positions (a list that grows block by block); token chunks beside them."""

    def __init__(self, cache_length: int, blocksize: int):
        self.cache_length, self.blocksize = cache_length, blocksize
        self.token_chunks = []
        self.blocks = []

    def append_token_chunk(self, chunk):  # keys_values/kvcache/base.py:844-855
        self.token_chunks.append(chunk.clone())

    def append_position_index(self, index: torch.Tensor, input_pos: int):  # :125-151
        bs = self.blocksize
        shape = index.shape[:2] + (bs,)
        bstart = (input_pos - self.cache_length) % bs
        if bstart == 0:
            self.blocks.append(torch.zeros(shape, dtype=torch.int64))
        block = self.blocks[-1]
        num = index.shape[2]
        bend = min(bstart + num, bs)
        iend = bend - bstart
        block[:, :, bstart:bend] = index[:, :, :iend]
        while iend < num:
            istart = iend
            block = torch.zeros(shape, dtype=torch.int64)
            self.blocks.append(block)
            bend = min(num - istart, bs)
            iend = istart + bend
            block[:, :, :bend] = index[:, :, istart:iend]

    def finalize(self, input_pos: int):  # :102-123: the last block cut to the positions in use
        if input_pos <= self.cache_length:
            return []
        end = (input_pos - self.cache_length) % self.blocksize
        if end == 0:
            return list(self.blocks)
        return self.blocks[:-1] + [self.blocks[-1][:, :, :end]]

    def extract_index(self, input_pos: int, num: int) -> torch.Tensor:  # :153-204
        assert input_pos >= self.cache_length
        pos, relpos, offset = self.cache_length, None, None
        for relpos, block in enumerate(self.blocks):
            if input_pos < pos + block.shape[-1]:
                offset = input_pos - pos
                break
            pos += block.shape[-1]
        assert offset is not None, "position too large"
        parts = []
        block = self.blocks[relpos]
        bend = min(offset + num, block.shape[-1])
        parts.append(block[:, :, offset:bend])
        done = bend - offset
        while done < num:
            relpos += 1
            block = self.blocks[relpos]
            bend = min(num - done, block.shape[-1])
            parts.append(block[:, :, :bend])
            done += bend
        return torch.cat(parts, dim=-1)


class PolicyCacheOracle:
    """One layer's cache with the step order of DefaultKVCache.forward
    (keys_values/kvcache/base.py:554-595): write (with the ring move) -> attend -> score -> select."""

    def __init__(self, B, Hq, Hkv, L, D, dtype=torch.bfloat16, max_chunk_size=None, grace_period=0, normalize_scores=False,
                 v_length=False, q_hitter=False, combination_constant=0.5, quantized=False, num_bits=8, replay_log_blocksize=None):
        assert 0 <= grace_period < L
        assert not q_hitter or quantized  # keys_values/kvcache/qh2o.py:95-96
        self.B, self.Hq, self.Hkv, self.L, self.D = B, Hq, Hkv, L, D
        self.dtype = dtype
        self.k = torch.zeros(B, Hkv, L, D, dtype=dtype)
        self.v = torch.zeros(B, Hkv, L, D, dtype=dtype)
        self.token_pos = torch.zeros(B, Hkv, L, dtype=torch.int32)
        self.buffers = {"scores": torch.zeros(B, Hkv, L, dtype=torch.float32)}
        if q_hitter:
            self.buffers["q_errors"] = torch.zeros(B, Hkv, L, dtype=torch.float32)
        if v_length:
            self.buffers["v_norm"] = torch.zeros(B, Hkv, L, dtype=torch.float32)
        self.max_chunk_size = None if (max_chunk_size is None or max_chunk_size > L // 2) else max_chunk_size  # :458-462
        self.grace_period = grace_period
        self.normalize_scores = normalize_scores
        self.v_length, self.q_hitter, self.c = v_length, q_hitter, combination_constant
        self.quantized = quantized
        self.num_bits = num_bits
        self.replay_log = ReplayLogOracle(L, replay_log_blocksize) if replay_log_blocksize else None
        self.input_pos = 0
        self.current_length = 0
        self.prefill_length = 0
        self.next_index = None
        self.next_grace_pos = None
        self.use_initial_rule = False
        self.scale = 1.0 / math.sqrt(D)

    @property
    def scores(self):
        return self.buffers["scores"]

    # -- what the store holds for a new row ---------------------------------------------------------

    def _stored(self, x: torch.Tensor) -> torch.Tensor:
        x = x.to(self.dtype)
        if not self.quantized:
            return x
        c, s, z = quantize_rows(x, self.num_bits)
        return dequantize_rows(c, s, z, self.dtype)

    def _initial_scores(self, key, value):
        """keys_values/kvcache/h2o.py:316-327 and keys_values/kvcache/qh2o.py:158-163."""
        init = {}
        if self.v_length:
            init["v_norm"] = torch.linalg.vector_norm(value, dim=-1, dtype=torch.float32)
        if self.q_hitter:
            init["q_errors"] = (quantization_error(key, self.num_bits).to(torch.float32)
                                + quantization_error(value, self.num_bits).to(torch.float32))
        return init

    # -- prefill (keys_values/kvcache/attn_weights.py:817-869) ---------------------------------------

    def prefill(self, query, key, value):
        n = key.shape[2]
        assert n <= self.L
        key, value = key.to(self.dtype), value.to(self.dtype)
        self.k[:, :, :n] = self._stored(key)
        self.v[:, :, :n] = self._stored(value)
        self.token_pos[:, :, :n] = torch.arange(n, dtype=torch.int32)
        for buf in self.buffers.values():
            buf.zero_()
        for name, vals in self._initial_scores(key, value).items():
            self.buffers[name][:, :, :n] = vals
        self.current_length = n
        self.prefill_length = n
        self.input_pos = n
        self.use_initial_rule = n == self.L
        self.next_index = None
        if self.grace_period > 0:
            self.next_grace_pos = self.L - self.grace_period
        o, _ = sdpa_in_blocks(query, key, value, self.scale, 0, None, return_attn_weights=False)
        return o

    # -- one step ------------------------------------------------------------------------------------

    def max_forward_length(self) -> int:
        """keys_values/kvcache/attn_weights.py:501-508."""
        diff = self.L - self.current_length
        result = self.L - self.grace_period
        if diff > 0:
            result = min(result, diff)
        if self.max_chunk_size is not None:
            result = min(result, self.max_chunk_size)
        return result

    def forward(self, query, key, value):
        num = key.shape[2]
        assert 1 <= num <= self.max_forward_length()
        B, Hkv, L, gp = self.B, self.Hkv, self.L, self.grace_period
        key, value = key.to(self.dtype), value.to(self.dtype)
        init = self._initial_scores(key, value)
        if self.current_length < L:  # free slots, attn_weights.py:1001-1016
            index = torch.arange(self.current_length, self.current_length + num).view(1, 1, -1).expand(B, Hkv, -1)
        elif self.use_initial_rule:  # :536-550
            n0 = min(int(KEEP_INITIAL_FRACTION * L), L - num)
            index = torch.arange(n0, n0 + num).view(1, 1, -1).expand(B, Hkv, -1)
            self.use_initial_rule = False
        else:
            index = self.next_index[:, :, :num]
        index = index.contiguous().to(torch.int64)
        gi = lambda idx: idx.unsqueeze(-1).expand(-1, -1, -1, self.D)  # noqa: E731
        cache_full = self.input_pos >= L
        if self.replay_log is not None and cache_full:  # attn_weights.py:629-633
            self.replay_log.append_position_index(index, self.input_pos)
        new_k, new_v = self._stored(key), self._stored(value)
        if cache_full and gp > 0:
            # attn_weights.py:267-303: token positions
            num2 = min(num, gp)
            num1 = num - num2
            prefix = L - gp
            pos_flat = positions_wrap_around(num2, self.next_grace_pos, prefix, L)
            positions = pos_flat.view(1, 1, -1).expand(B, Hkv, -1)
            self.token_pos[:, :, pos_flat] = torch.arange(self.input_pos + num1, self.input_pos + num, dtype=torch.int32)
            new_tps = torch.arange(self.input_pos - gp, self.input_pos - gp + num, dtype=torch.int32)
            self.token_pos.scatter_(-1, index, new_tps.view(1, 1, -1).expand(B, Hkv, -1))
            # :578-590: [ring rows | new rows] go to [index | ring slots]
            # the ring rows come out of the dequantised buffer and go through the same write as the new
            # rows, which quantises them again (keys_values/kvcache/quant_buffers.py:732-775)
            key_cp = torch.cat((self._stored(self.k.gather(-2, gi(positions))), new_k), dim=-2)
            value_cp = torch.cat((self._stored(self.v.gather(-2, gi(positions))), new_v), dim=-2)
            fused = torch.cat((index, positions), dim=-1)
            self.k.scatter_(-2, gi(fused), key_cp)
            self.v.scatter_(-2, gi(fused), value_cp)
            # :645-677: score buffers
            for name, buf in self.buffers.items():
                src = buf[:, :, pos_flat]
                vals = init.get(name)
                if num1 > 0:
                    part2 = vals[:, :, :num1] if vals is not None else torch.zeros(B, Hkv, num1)
                    src = torch.cat((src, part2), dim=-1)
                buf.scatter_(-1, index, src)
                buf[:, :, pos_flat] = 0.0 if vals is None else vals[:, :, num1:]
            if num1 == 0:  # :601-606
                self.next_grace_pos = (self.next_grace_pos - prefix + num) % gp + prefix
        else:
            new_tps = torch.arange(self.input_pos, self.input_pos + num, dtype=torch.int32)
            self.token_pos.scatter_(-1, index, new_tps.view(1, 1, -1).expand(B, Hkv, -1))
            self.k.scatter_(-2, gi(index), new_k)
            self.v.scatter_(-2, gi(index), new_v)
            for name, buf in self.buffers.items():  # :678-681
                vals = init.get(name)
                if vals is None:
                    buf.scatter_(-1, index, 0.0)
                else:
                    buf.scatter_(-1, index, vals)
        if self.current_length < L:
            self.current_length += num
        T = self.current_length
        o, w = sdpa_in_blocks(query, self.k[:, :, :T], self.v[:, :, :T], self.scale, self.input_pos,
                              self.token_pos[:, :, :T].to(torch.int64))
        self.input_pos += num
        self._update(w, num)
        return o, w, index

    def _update(self, w: torch.Tensor, query_length: int):
        T, L = self.current_length, self.L
        full = T == L
        limit = L - self.grace_period if full else T
        k = limit if self.max_chunk_size is None else self.max_chunk_size
        nxt, compared = update_select(
            self.scores, w, T, limit, k if full else 1, normalize=self.normalize_scores and full, token_pos=self.token_pos,
            input_pos=self.input_pos, prefill_len=self.prefill_length, v_norm=self.buffers.get("v_norm"),
            q_errors=self.buffers.get("q_errors") if full else None, combination=self.c, q_len=query_length)
        self.next_index = nxt if full else None
        self.compared = compared
