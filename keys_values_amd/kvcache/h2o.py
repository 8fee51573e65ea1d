"""
``H2OKVCache``: the heavy-hitter-oracle cache of the reference on the HIP kernels, with the call
surface of ``DefaultKVCache`` / ``AttnWeightsKVCache`` / ``H2OKVCache``
(keys_values/kvcache/base.py:554-595, keys_values/kvcache/attn_weights.py:325-1029,
keys_values/kvcache/h2o.py:28-263): ``forward(query, key, value, token_idx)``, ``next_positions``,
``token_positions``, ``max_forward_length``, ``_update``, the buffers ``token_pos`` (int32),
``scores`` (float32) and the K/V buffers ``(max_batch, n_query_groups, cache_length, head_size)``.

One ``forward`` is, in the reference's order (keys_values/kvcache/base.py:554-595): write the new
tokens into the slots chosen last time (resetting their score), attend over the cache with the
position mask, add the score-sums to the cumulative scores, choose the next slots to evict.

The K/V store is either bf16 (``h2o-default``) or codes with per-row scale / zero point: 8 bits
(``h2o-torch-quantized8``) or 4 bits, two codes per byte (``h2o-torch-quantized4``;
keys_values/kvcache/factory.py:50-66). In the second case the codes stay resident and are never
written back: single tokens and short chunks are attended to by kernels that dequantise on load; for a
long chunk (``dequantize_chunk_rows`` query rows or more) the store is dequantised once into a bf16
buffer shared by all caches of a device and stream, because every workgroup of the attention kernels
would otherwise dequantise the whole store again. The reference dequantises the whole cache into a
bf16 working buffer per layer and re-quantises it afterwards
(keys_values/kvcache/quant_buffers.py:473-503,732-804).

Policy variants on the same kernels: a grace period (the last ``grace_period`` slots are a ring of
the most recent tokens, never evicted; keys_values/kvcache/attn_weights.py:267-303,565-606), the
V-norm weighted instantaneous score (``VLengthH2OKVCache``, keys_values/kvcache/h2o.py:266-420) and
the Q-Hitter combination with the quantisation error (``QuantizedH2OKVCache`` /
``QuantizedVLengthH2OKVCache``, keys_values/kvcache/qh2o.py). ``create_kv_cache`` takes the names of
keys_values/kvcache/factory.py:50-66. With ``switch_replay_logging(True)`` the cache records the token
chunks and the slot every later token went to (keys_values/kvcache/attn_weights.py:43-204,939-966).

With ``blocks_over_heads=True`` (keys_values/kvcache/quant_buffers.py:849-870) a quantisation block is a slot
over all heads. The cache then works the way the reference's quantised buffers do
(keys_values/kvcache/quant_buffers.py:361-804): the codes live in two block stores, the kernels run on a
dequantised working buffer shared by the caches of a device and stream (a cache that finds the buffer holding
another cache's rows dequantises its own store into it first), and after every slot write the touched slots are
quantised again as whole blocks from the working rows and read back, so that the buffer always holds what the
codes say. Every policy variant runs on it; the quantisation errors of the Q-Hitter combination are those of the new
tokens' blocks over the heads (keys_values/kvcache/quant_buffers.py:306-331).

Not covered (raises): fp32 caches, bitsandbytes stores.
"""
import ctypes
import weakref
from dataclasses import dataclass
from typing import Optional

import torch

from .. import _lib
from ..attention import ops
from .quantize import RowQuantizer
from .replay import DEFAULT_REPLAY_LOG_BLOCKSIZE, AttnWeightsReplayLog, ReplayArena

DEFAULT_KEEP_INITIAL_FRACTION = 0.05  # keys_values/kvcache/attn_weights.py:322
DEFAULT_COMBINATION_CONSTANT = 0.5  # keys_values/kvcache/qh2o.py:25
# Slots one launch of the selection kernel chooses. A step on a full cache chooses min(this, what the
# cache may be asked for); a later request for more (a chunk longer than this with no max_chunk_size) is
# served by selecting again, from the same scores, as many slots as it needs.
EAGER_SELECT = 4096
# Query rows (tokens x heads per KV head) of a chunk from which dequantising the store once per chunk
# is faster than dequantising it inside the attention kernels (every 256 rows walk the whole store):
# the copy costs two passes over the store, the kernels gain in proportion to the rows.
DEFAULT_DEQUANTIZE_CHUNK_ROWS = 2048

_dequant_buffers = {}
_dequant_owner = {}  # per buffer: the cache whose rows it holds as that cache's working buffer (blocks over heads), else None


def _dequant_scratch(device, numel: int, dtype: torch.dtype = torch.bfloat16, owner=None):
    """Two 16-bit buffers of ``numel`` elements of ``dtype``, grow-only, shared by the caches of one device and
    stream (launches on a stream are ordered: a layer's attention has read them before the next layer's
    dequantisation overwrites them). ``owner``: the cache that is about to use them as its working buffer; the third
    value returned says whether they still hold that cache's rows from its last use. Any other use takes the
    buffers away from their owner."""
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    buf = _dequant_buffers.get(key)
    fresh = buf is None or buf.numel() < 2 * numel
    if fresh:
        buf = torch.empty(2 * numel, dtype=torch.int16, device=device)
        _dequant_buffers[key] = buf
    before = _dequant_owner.get(key)
    held = (not fresh) and owner is not None and before is not None and before[0]() is owner and before[1] == numel
    if before is not None and before[0]() is not None and before[0]() is not owner:
        before[0]().wait_for_selection()  # its second stream may still be reading the rows
    _dequant_owner[key] = (weakref.ref(owner), numel) if owner is not None else None
    buf = buf.view(dtype)
    return buf[:numel], buf[numel : 2 * numel], held


@dataclass(frozen=True)
class KVCacheParams:
    """keys_values/kvcache/base.py:29-66."""

    max_batch_size: int
    n_query_groups: int
    cache_length: int
    head_size: int
    n_head: int
    dtype: Optional[torch.dtype] = torch.bfloat16


class H2OKVCache:
    def __init__(
        self,
        params: KVCacheParams,
        max_chunk_size: Optional[int] = None,
        normalize_scores: bool = False,
        grace_period: int = 0,
        quantized: bool = False,
        num_bits: int = 8,
        keep_initial_fraction: float = DEFAULT_KEEP_INITIAL_FRACTION,
        device: Optional[torch.device] = None,
        v_length: bool = False,
        q_hitter: bool = False,
        combination_constant: float = DEFAULT_COMBINATION_CONSTANT,
        replay_log_blocksize: Optional[int] = None,
        overlap_select: bool = False,
        dequantize_chunk_rows: Optional[int] = DEFAULT_DEQUANTIZE_CHUNK_ROWS,
        blocks_over_heads: bool = False,
    ):
        self._init_kwargs = dict(max_chunk_size=max_chunk_size, normalize_scores=normalize_scores, grace_period=grace_period,
                                 quantized=quantized, num_bits=num_bits, keep_initial_fraction=keep_initial_fraction, device=device,
                                 v_length=v_length, q_hitter=q_hitter, combination_constant=combination_constant,
                                 replay_log_blocksize=replay_log_blocksize, overlap_select=overlap_select,
                                 dequantize_chunk_rows=dequantize_chunk_rows, blocks_over_heads=blocks_over_heads)
        # blocks_over_heads (quantised stores only): one quantisation block per slot over all heads; see the module text
        self.blocks_over_heads = bool(blocks_over_heads) and quantized
        # dequantize_chunk_rows: a chunk with at least this many query rows (tokens x heads per KV head) is
        # attended to over a bf16 copy of the quantised store made once for the chunk; None = never.
        self.dequantize_chunk_rows = dequantize_chunk_rows
        # overlap_select: launch the score update + eviction choice of a chunk step (and, for a long chunk over
        # a quantised store, the score-sum pass before them) on a second stream, so
        # that it runs beside whatever the caller enqueues next; the next forward and next_positions() wait
        # for it. The attributes scores, token_pos and _next_index are plain tensors: a caller that reads
        # them directly calls wait_for_selection() first.
        self._overlap = bool(overlap_select)
        self._side_stream = None
        self._select_done = None
        self._select_keep = None
        if replay_log_blocksize is None:  # keys_values/kvcache/attn_weights.py:436-441
            replay_log_blocksize = DEFAULT_REPLAY_LOG_BLOCKSIZE
        elif replay_log_blocksize <= 0:
            raise ValueError(f"replay_log_blocksize must be positive, but got {replay_log_blocksize}")
        self.replay_log_blocksize = replay_log_blocksize
        self._log_on = False        # switch_replay_logging
        self._log_chunks = None     # token chunks since the last prefill (None until a prefill was logged)
        self._log_arena = None
        if not (0 <= grace_period < params.cache_length):  # keys_values/kvcache/attn_weights.py:440-444
            raise ValueError(f"grace_period = {grace_period}, must be in [0, {params.cache_length})")
        if num_bits not in (4, 8):  # keys_values/kvcache/quantize/pytorch.py:191-192
            raise ValueError(f"num_bits = {num_bits}, must be 4 or 8")
        if q_hitter and not quantized:  # keys_values/kvcache/qh2o.py:95-96
            raise TypeError("the quantisation-error policy needs the quantised store")
        if not (0 <= combination_constant <= 1):  # keys_values/kvcache/qh2o.py:97-100
            raise ValueError(f"combination_constant = {combination_constant}, must be in [0, 1]")
        if params.dtype not in (None, torch.bfloat16, torch.float16):
            raise NotImplementedError(f"cache dtype {params.dtype}: the kernels take bfloat16 or float16")
        if params.head_size not in (ops.QUANTIZED_HEAD_SIZES if quantized else ops.ALLOWED_HEAD_SIZES):
            raise NotImplementedError(f"head_size = {params.head_size} not in {ops.QUANTIZED_HEAD_SIZES if quantized else ops.ALLOWED_HEAD_SIZES}")
        if params.n_head % params.n_query_groups != 0:
            raise ValueError("n_head must be a multiple of n_query_groups")
        self.params = params
        self.max_batch_size = params.max_batch_size
        self.n_query_groups = params.n_query_groups
        self.n_head = params.n_head
        self.cache_length = params.cache_length
        self.head_size = params.head_size
        self.dtype = params.dtype if params.dtype is not None else torch.bfloat16
        self.grace_period = grace_period
        self.next_grace_pos = None
        self.v_length = v_length
        self.q_hitter = q_hitter
        self.combination_constant = combination_constant
        self.normalize_scores = normalize_scores
        self.quantized = quantized
        self.num_bits = num_bits if quantized else None
        # keys_values/kvcache/attn_weights.py:458-462: silently disabled when too large
        if max_chunk_size is not None and max_chunk_size > self.cache_length // 2:
            max_chunk_size = None
        self.max_chunk_size = max_chunk_size
        limit = self.cache_length - grace_period
        # what next_positions may be asked for on a full cache: the whole argsort when no chunk size is set
        # (keys_values/kvcache/attn_weights.py:773-783)
        self._select_k = limit if max_chunk_size is None else min(max_chunk_size, limit)
        self._next_count = 0  # leading entries of _next_index that hold the current choice
        self._keep_initial_fraction = keep_initial_fraction
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        if self.device.type != "cuda":
            raise RuntimeError(f"H2OKVCache buffers live on a ROCm device, not on {self.device}: there is no CPU path")
        b, h, length, d = self.max_batch_size, self.n_query_groups, self.cache_length, self.head_size
        kv_dtype = torch.uint8 if quantized else self.dtype
        row = d // 2 if (quantized and num_bits == 4) else d  # the 4-bit store packs two codes per byte
        if self.blocks_over_heads:
            # the codes; k and v are bound to the shared working buffer by every forward (_bind_working)
            self.block_store_k = RowQuantizer((b, h, length, d), self.dtype, num_bits, True, allocate_buffers=True, device=self.device)
            self.block_store_v = RowQuantizer((b, h, length, d), self.dtype, num_bits, True, allocate_buffers=True, device=self.device)
            for q in (self.block_store_k, self.block_store_v):
                q.quant_buffer.zero_()
            self.k = self.v = None
        else:
            # K and V (and their row states) are the two halves of one allocation each: one launch can walk both
            self._kv = torch.zeros((2, b, h, length, row), dtype=kv_dtype, device=self.device)  # buffers.py:462-464
            self.k, self.v = self._kv[0], self._kv[1]
        if quantized and not self.blocks_over_heads:
            self._kv_scale = torch.zeros((2, b, h, length), dtype=torch.float32, device=self.device)
            self._kv_zp = torch.zeros((2, b, h, length), dtype=torch.int32, device=self.device)
            self.k_scale, self.v_scale = self._kv_scale[0], self._kv_scale[1]
            self.k_zp, self.v_zp = self._kv_zp[0], self._kv_zp[1]
        self.token_pos = torch.zeros((b, h, length), dtype=torch.int32, device=self.device)  # attn_weights.py:466-470
        self.scores = torch.zeros((b, h, length), dtype=torch.float32, device=self.device)  # h2o.py:85-91
        # further score buffers, moved and initialised with the slots (h2o.py:405-413, qh2o.py:107-113)
        self.v_norm = torch.zeros((b, h, length), dtype=torch.float32, device=self.device) if v_length else None
        self.q_errors = torch.zeros((b, h, length), dtype=torch.float32, device=self.device) if q_hitter else None
        if grace_period > 0:  # the ring twice over: any wrap-around run of up to grace_period slots is one view of it
            ring = torch.arange(length - grace_period, length, dtype=torch.int32, device=self.device)
            self._ring_twice = torch.cat((ring, ring))
        # the current choice: (batch, heads, _next_count) slots, packed at the start of this buffer
        self._next_flat = torch.zeros(b * h * self._select_k, dtype=torch.int32, device=self.device)
        self._have_next = False
        self._use_initial_rule = None
        self._input_pos = 0
        self.batch_size = None
        self.current_length = None
        self.prefill_length = None
        self.scale_factor = 1.0 / (self.head_size ** 0.5)

    # -- bookkeeping -----------------------------------------------------------------------------

    @property
    def input_pos(self) -> int:
        return self._input_pos

    @property
    def max_prefill_length(self) -> int:
        return self.cache_length  # keys_values/kvcache/base.py:707-709

    def max_forward_length(self) -> int:
        """keys_values/kvcache/attn_weights.py:501-508."""
        diff = self.cache_length - self.current_length
        result = self.cache_length - self.grace_period
        if diff > 0:
            result = min(result, diff)
        if self.max_chunk_size is not None:
            result = min(result, self.max_chunk_size)
        return result

    def token_positions(self) -> torch.Tensor:
        if self.current_length is None:
            raise IndexError("Cache is not initialized, call 'prefill' first")
        return self.token_pos[: self.batch_size, :, : self.current_length]

    # -- the rest of the reference's cache surface (keys_values/kvcache/base.py:249-377,669-712) ------------

    def reset(self) -> None:
        """``input_pos == 0`` afterwards: the next ``forward`` is the prefill of a new sequence
        (keys_values/kvcache/base.py:343-350,700-702)."""
        self.wait_for_selection()
        self._input_pos = 0
        self._have_next = False

    def update_requires_attn_weights(self) -> bool:
        return True  # keys_values/kvcache/attn_weights.py: the H2O family scores slots by attention weights

    def get_params(self) -> KVCacheParams:
        return KVCacheParams(self.max_batch_size, self.n_query_groups, self.cache_length, self.head_size, self.n_head, self.dtype)

    def get_keys_values(self):
        """A ``KeysAndValues`` holder over the slots in use, or None before the first prefill
        (keys_values/kvcache/base.py:249-257). Quantised stores hand out holders that dequantise on ``keys()`` /
        ``values()``."""
        from .buffers import BlockQuantizedKeysAndValues, DefaultKeysAndValues, QuantizedKeysAndValues

        if self.batch_size is None or self.current_length is None or self._input_pos == 0:
            return None
        self.wait_for_selection()
        b, t = self.batch_size, self.current_length
        if self.blocks_over_heads:
            for q in (self.block_store_k, self.block_store_v):
                q.allocate_buffers(b)
            return BlockQuantizedKeysAndValues(self.block_store_k, self.block_store_v, b, t)
        if not self.quantized:
            return DefaultKeysAndValues(self.k[:b, :, :t], self.v[:b, :, :t])
        return QuantizedKeysAndValues(self.k[:b, :, :t], self.v[:b, :, :t], self._quant_state(t), self.head_size, self.num_bits, self.dtype)

    def get_v_norm(self) -> torch.Tensor:
        """Norms of the stored V rows, (batch, n_query_groups, current_length) (keys_values/kvcache/h2o.py:273-283)."""
        if self.v_norm is None:
            raise AttributeError("this cache does not weight its scores by the V norms")
        if self.current_length is None:
            raise IndexError("Cache is not initialized, call 'prefill' first")
        return self.v_norm[: self.batch_size, :, : self.current_length]

    def size_estimate(self):
        """(bits in total, bits by part) of the buffers this cache holds (keys_values/kvcache/attn_weights.py:900-909,
        keys_values/kvcache/h2o.py:235-242). The working buffer that caches with blocks over the heads share is not
        counted: it belongs to the device, not to a cache."""
        def bits(*ts):
            return 8 * sum(t.numel() * t.element_size() for t in ts if t is not None)

        if self.blocks_over_heads:
            qs = (self.block_store_k, self.block_store_v)
            parts = {"buffers": bits(*(q.quant_buffer for q in qs)), "quant_state": bits(*(t for q in qs for t in (q.quant_scales, q.quant_zero_points)))}
        elif self.quantized:
            parts = {"buffers": bits(self._kv), "quant_state": bits(self._kv_scale, self._kv_zp)}
        else:
            parts = {"buffers": bits(self._kv)}
        parts["token_pos"] = bits(self.token_pos)
        score_parts = {"scores": self.scores, "v_norm": self.v_norm, "q_errors": self.q_errors}
        total_scores = 0
        for name, t in score_parts.items():
            if t is not None:
                total_scores += bits(t)
                if name != "scores":
                    parts[name] = bits(t)
        parts["scores"] = total_scores  # all score buffers together, as the reference reports them
        return sum(v for k, v in parts.items() if k not in ("v_norm", "q_errors")), parts

    @classmethod
    def size_estimate_apriori(cls, params: KVCacheParams, **kwargs):
        """The same without a cache (keys_values/kvcache/attn_weights.py:911-937, keys_values/kvcache/h2o.py:244-255).
        ``kwargs`` as the constructor's: ``quantized``, ``num_bits``, ``blocks_over_heads``, ``v_length``, ``q_hitter``."""
        if params.dtype is None:
            raise ValueError("params.dtype must be provided")
        rows = params.max_batch_size * params.n_query_groups * params.cache_length
        quantized, num_bits = kwargs.get("quantized", False), kwargs.get("num_bits", 8)
        if quantized:
            states = params.max_batch_size * params.cache_length if kwargs.get("blocks_over_heads") else rows
            parts = {"buffers": 2 * rows * params.head_size * num_bits, "quant_state": 2 * states * 64}
        else:
            parts = {"buffers": 2 * rows * params.head_size * 8 * torch.empty((), dtype=params.dtype).element_size()}
        parts["token_pos"] = rows * 32
        n_scores = 1 + int(bool(kwargs.get("v_length"))) + int(bool(kwargs.get("q_hitter")))
        if kwargs.get("v_length"):
            parts["v_norm"] = rows * 32
        if kwargs.get("q_hitter"):
            parts["q_errors"] = rows * 32
        parts["scores"] = n_scores * rows * 32
        return sum(v for k, v in parts.items() if k not in ("v_norm", "q_errors")), parts

    def clone(self) -> "H2OKVCache":
        """A new, empty cache with this one's settings (keys_values/kvcache/base.py:364-377: buffers are not copied)."""
        return type(self)(self.params, **self._init_kwargs)

    def _second_stream(self) -> torch.cuda.Stream:
        if self._side_stream is None:
            self._side_stream = torch.cuda.Stream(self.device)  # default priority
        return self._side_stream

    def wait_for_selection(self):
        """Make the caller's stream wait for an eviction choice still running on the second stream."""
        if self._select_done is not None:
            torch.cuda.current_stream(self.device).wait_event(self._select_done)
            self._select_done, self._select_keep = None, None

    @property
    def _next_index(self) -> torch.Tensor:
        """(max_batch_size, n_query_groups, _next_count) view of the slots chosen last."""
        c = max(self._next_count, 1)
        n = self.max_batch_size * self.n_query_groups * c
        return self._next_flat[:n].view(self.max_batch_size, self.n_query_groups, c)

    def set_next_positions(self, index: torch.Tensor):
        """Replace the choice of the next slots to write by ``index`` (batch, n_query_groups, num): for
        callers that decide the eviction themselves, and for tests that keep two caches in step."""
        b, h, num = index.shape
        if h != self.n_query_groups or b > self.max_batch_size or not 1 <= num <= self._select_k:
            raise ValueError(f"index.shape = {tuple(index.shape)} does not fit the cache")
        self.wait_for_selection()
        self._next_count = num
        self._next_index[:b].copy_(index.to(device=self.device, dtype=torch.int32))
        self._have_next = True

    def next_positions(self, num: int) -> Optional[torch.Tensor]:
        """Slots the next ``forward`` writes to, int64 (batch, n_query_groups, num), or None
        (keys_values/kvcache/attn_weights.py:490-499)."""
        self.wait_for_selection()
        idx = self._next_index_for(num, peek=True)
        return None if idx is None else idx.to(torch.int64)

    # -- replay log (keys_values/kvcache/attn_weights.py:939-966) ---------------------------------------

    def switch_replay_logging(self, status: bool):
        self._log_on = bool(status)
        if not status:
            self._log_chunks, self._log_arena = None, None

    @property
    def do_replay_logging(self) -> bool:
        return self._log_on

    def get_replay_log(self) -> Optional[AttnWeightsReplayLog]:
        """Token chunks and, for every token position >= cache_length, the slot it was written to."""
        if not self._log_on:
            return None
        if self._log_chunks is None:
            raise IndexError("Cannot switch on replay logging in the middle of inference run. Call 'prefill'.")
        positions = max(self._input_pos - self.cache_length, 0)
        blocks = self._log_arena.blocks(positions) if positions > 0 else []
        return AttnWeightsReplayLog(list(self._log_chunks), blocks, self.cache_length, self.max_prefill_length,
                                    self.replay_log_blocksize, self.grace_period)

    def _log_token_chunk(self, token_idx: Optional[torch.Tensor], num: int, prefill: bool):
        if not self._log_on:
            return
        if prefill:  # keys_values/kvcache/attn_weights.py:865-868: a prefill starts a new log
            self._log_chunks = []
            self._log_arena = ReplayArena(self.batch_size, self.n_query_groups, self.replay_log_blocksize, self.device)
        elif self._log_chunks is None:  # :623-628
            raise IndexError("Cannot switch on replay logging in the middle of inference run. Call 'prefill'.")
        if token_idx is None or tuple(token_idx.shape) != (self.batch_size, num):
            raise ValueError(f"token_idx must be given with shape {(self.batch_size, num)} while the replay log is on")
        self._log_chunks.append(token_idx.detach().clone())  # keys_values/kvcache/base.py:844-855

    def _quant_state(self, T: int) -> Optional[ops.QuantState]:
        if not self.quantized or self.blocks_over_heads:  # blocks over heads: the kernels read the working buffer
            return None
        b = self.batch_size
        return ops.QuantState(self.k_scale[:b, :, :T], self.k_zp[:b, :, :T], self.v_scale[:b, :, :T], self.v_zp[:b, :, :T])

    def _next_index_for(self, num: int, peek: bool = False) -> Optional[torch.Tensor]:
        b, h = self.batch_size, self.n_query_groups
        if self.current_length is None:
            return None
        if self.current_length < self.cache_length:  # free slots, attn_weights.py:1001-1016
            start = self.current_length
            return torch.arange(start, start + num, dtype=torch.int32, device=self.device).view(1, 1, -1).expand(b, h, -1).contiguous()
        if self._use_initial_rule:  # attn_weights.py:536-550
            n0 = min(int(self._keep_initial_fraction * self.cache_length), self.cache_length - num)
            # with a grace period the evicted slots must stay below the ring (the reference's formula
            # does not look at it; it only matters for chunks nearly as long as the evictable part)
            n0 = min(n0, self.cache_length - self.grace_period - num)
            if not peek:
                self._use_initial_rule = False
            return torch.arange(n0, n0 + num, dtype=torch.int32, device=self.device).view(1, 1, -1).expand(b, h, -1).contiguous()
        if not self._have_next:
            return None
        if num > self._next_count:
            self._select_more(num)
        return self._next_index[:b, :, :num]

    def _select_more(self, num: int):
        """The step before chose fewer slots than are asked for now (it could not know): choose ``num`` from
        the same scores. Nothing is added to them (no weights), so the first entries come out as before."""
        if num > self._select_k:
            raise ValueError(f"num = {num} exceeds what a full cache hands out ({self._select_k})")
        a = self._h2o_args(True, num)
        a.next_index = self._next_flat.data_ptr()
        lib = _lib.load()
        with torch.cuda.device(self.device):
            nbytes = lib.kvx_h2o_workspace_bytes(ctypes.byref(a))
            ws = _lib.workspace(self.device, nbytes)
            a.workspace = _lib.ptr(ws)
            a.workspace_bytes = 0 if ws is None else ws.numel()
            _lib.check(lib.kvx_h2o_update_select(ctypes.byref(a), _lib.stream_ptr(self.device)))
        self._next_count = num

    # -- the step (keys_values/kvcache/base.py:554-595) -----------------------------------------

    def forward(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, token_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        """query (B, n_head, num, hs); key/value (B, n_query_groups, num, hs). Returns the attention
        output (B, num, n_head * hs) (keys_values/attention/base.py:378-380)."""
        _lib.require_gpu(query, key, value)
        if query.ndim != 4 or key.ndim != 4 or key.shape != value.shape:
            raise ValueError("query, key, value must be 4D and key.shape == value.shape")
        b, hq, num, d = query.shape
        if key.shape != (b, self.n_query_groups, num, d) or hq != self.n_head or d != self.head_size:
            raise ValueError(f"shapes {tuple(query.shape)}, {tuple(key.shape)} do not fit the cache")
        input_pos = self._input_pos
        self.wait_for_selection()
        if self.blocks_over_heads:
            self._bind_working(fresh=input_pos == 0)
        if input_pos == 0:
            out = self._prefill_step(query, key, value)
            self._log_token_chunk(token_idx, num, prefill=True)
            return out
        if b != self.batch_size:
            raise ValueError(f"batch size {b} differs from the prefill batch size {self.batch_size}")
        if self._use_initial_rule is None:
            raise IndexError("Cache needs to be initialized with 'prefill' before being used")
        diff = self.cache_length - self.current_length
        if not 1 <= num <= self.max_forward_length():
            if 0 < diff < num:
                raise ValueError(f"key.shape[2] = {num}, must be <= {diff} as long as the cache is not full")
            raise ValueError(f"key.shape[2] = {num}, must be in [1, {self.max_forward_length()}]")
        index = self._next_index_for(num)
        if index is None:
            raise IndexError("Cache needs to be initialized with 'prefill' before being used")
        self._log_token_chunk(token_idx, num, prefill=False)
        ring = self._write(index, key, value, input_pos)
        if self.blocks_over_heads:
            self._block_errors(index, ring, key, value)
            self._write_back(index, ring, (self.current_length, self.current_length + num) if diff > 0 else None)
        if diff > 0:
            self.current_length += num
        self._have_next = False
        self._input_pos += num
        T = self.current_length
        kc, vc = self.k[:b, :, :T], self.v[:b, :, :T]
        tp = self.token_pos[:b, :, :T]
        quant = self._quant_state(T)
        if num == 1 and T == self.cache_length:
            # one token into a full cache: attention, score update and eviction choice in one call
            out = self._decode_h2o_step(query, kc, vc, quant).unsqueeze(1)
            return out.reshape(b, num, hq * d)
        if num == 1:
            out, w, _ = ops.decode_core(query, kc, vc, self.scale_factor, return_weights=True, quant=quant)
            out = out.unsqueeze(1)
        else:
            rows = num * (hq // self.n_query_groups)
            if quant is not None and self.dequantize_chunk_rows is not None and rows >= self.dequantize_chunk_rows:
                # attention over the bf16 copy; the score-sum pass keeps the codes (it dequantises each key
                # once per wavefront whatever the chunk length, and reads half the bytes)
                kd, vd = self._dequantized(b, T)
                out, _, lse = ops.prefill_core(query, kd, vd, self.scale_factor, input_pos, tp, return_lse=True, output_transposed=True)
                if self._overlap:
                    # the score-sum pass too runs beside the caller's next launches: nothing needs the score-sums
                    # before the next chunk's eviction choice
                    main = torch.cuda.current_stream(self.device)
                    side = self._second_stream()
                    ready = torch.cuda.Event()
                    ready.record(main)
                    with torch.cuda.stream(side):
                        side.wait_event(ready)
                        w = ops.score_sum_core(query, kc, lse, self.scale_factor, input_pos, tp, quant=quant)
                        self._update(w, num)
                    query.record_stream(side)
                    lse.record_stream(side)
                    return out.reshape(b, num, hq * d)
                w = ops.score_sum_core(query, kc, lse, self.scale_factor, input_pos, tp, quant=quant)
            else:
                out, w, _ = ops.prefill_core(query, kc, vc, self.scale_factor, input_pos, tp, return_weights=True,
                                             output_transposed=True, quant=quant)
        self._update(w, num)
        return out.reshape(b, num, hq * d)

    __call__ = forward

    # -- blocks over the heads: working buffer and write-back (keys_values/kvcache/quant_buffers.py:473-503,732-804) --

    def _bind_working(self, fresh: bool):
        """Point k / v at the shared working buffer and make it hold this cache's rows: dequantise the block stores
        into it unless it still holds them from this cache's last step (``fresh``: a new sequence starts, nothing
        stored counts)."""
        bmax, h, length, d = self.max_batch_size, self.n_query_groups, self.cache_length, self.head_size
        kd, vd, held = _dequant_scratch(self.device, bmax * h * length * d, self.dtype, owner=self)
        self.k, self.v = kd.view(bmax, h, length, d), vd.view(bmax, h, length, d)
        if fresh or held or self.batch_size is None:
            return
        b = self.batch_size
        for q, work in ((self.block_store_k, self.k), (self.block_store_v, self.v)):
            q.allocate_buffers(b)
            q.dequantize(0, length, out=work[:b])

    def _block_errors(self, index: torch.Tensor, ring: Optional[torch.Tensor], key: torch.Tensor, value: torch.Tensor):
        """Quantisation errors of the new tokens for the Q-Hitter combination (keys_values/kvcache/qh2o.py:130-160):
        with blocks over the heads they are those of the new tokens' own blocks, one per token over all heads
        (keys_values/kvcache/quant_buffers.py:306-331), which the row-quantising slot write cannot produce. With a
        grace period the errors of the ring slots move out with their rows first (``index[..., :num2]``), the last
        ``num2`` new tokens then take the ring slots (keys_values/kvcache/attn_weights.py:267-303)."""
        if self.q_errors is None:
            return
        b, h, num = index.shape
        err = self.block_store_k.quantization_error(key.to(self.dtype)) + self.block_store_v.quantization_error(value.to(self.dtype))
        slots = index.long()
        if ring is not None:
            num2 = ring.numel()
            rs = ring.long().view(1, 1, num2).expand(b, h, num2)
            self.q_errors[:b].scatter_(2, slots[:, :, :num2], self.q_errors[:b].gather(2, rs))
            slots = torch.cat((slots[:, :, num2:], rs), dim=2)
        self.q_errors[:b].scatter_(2, slots, err)

    def _write_back(self, index: torch.Tensor, ring: Optional[torch.Tensor], span):
        """Quantise the slots just written as whole blocks from the working rows and read them back. ``span``: the
        slot range when every head wrote the same slots (prefill, filling); else the slots are ``index`` (batch,
        heads, num) and the ring slots that took new tokens. A slot that several heads wrote is processed once per
        head, with the same result every time: no host synchronisation to find the distinct ones."""
        b, h, length, d = self.batch_size, self.n_query_groups, self.cache_length, self.head_size
        stores = ((self.block_store_k, self.k), (self.block_store_v, self.v))
        for q, _ in stores:
            q.allocate_buffers(b)
        if span is not None:
            start, end = span
            for q, work in stores:
                q.quantize(start, end, work[:b, :, start:end])
                work[:b, :, start:end] = q.dequantize(start, end)
            return
        slots = index.reshape(b, -1).long()
        if ring is not None:
            slots = torch.cat((slots, ring.long().view(1, -1).expand(b, -1)), dim=1)
        n = slots.shape[1]
        blocks = (torch.arange(b, device=self.device).view(b, 1) * length + slots).reshape(-1)  # flat (batch, slot) ids
        gi = slots.view(b, 1, n, 1).expand(b, h, n, d)
        for q, work in stores:
            tmp = RowQuantizer((b, h, n, d), self.dtype, self.num_bits, True, allocate_buffers=True, device=self.device)
            tmp.quantize(0, n, work[:b].gather(2, gi))
            q.quant_buffer.view(-1, q.quant_buffer.shape[-1])[blocks] = tmp.quant_buffer.view(b * n, -1)
            q.quant_scales.view(-1)[blocks] = tmp.quant_scales.view(-1)
            q.quant_zero_points.view(-1)[blocks] = tmp.quant_zero_points.view(-1)
            work[:b].scatter_(2, gi, tmp.dequantize(0, n))

    def _dequantized(self, b: int, T: int):
        """bf16 views (b, n_query_groups, T, head_size) of the quantised store, dequantised into the shared
        scratch by one launch per tensor (all slots of the first ``b`` batch entries: they are contiguous)."""
        h, length, d = self.n_query_groups, self.cache_length, self.head_size
        rows = b * h * length
        kd, vd, _ = _dequant_scratch(self.device, rows * d, self.dtype)
        lib = _lib.load()
        bits, elem = self.num_bits, _lib.elem_kv_dtype(self.dtype)

        def fn(c, s, z, n, dd, o, stride, stream):
            return lib.kvx_dequantize_rows_typed(c, s, z, n, dd, bits, elem, o, stride, stream)

        with torch.cuda.device(self.device):
            stream = _lib.stream_ptr(self.device)
            if b == self.max_batch_size:  # K and V are adjacent in the store and in the scratch: one launch
                _lib.check(fn(self._kv.data_ptr(), self._kv_scale.data_ptr(), self._kv_zp.data_ptr(), 2 * rows, d, kd.data_ptr(), d, stream))
            else:
                _lib.check(fn(self.k.data_ptr(), self.k_scale.data_ptr(), self.k_zp.data_ptr(), rows, d, kd.data_ptr(), d, stream))
                _lib.check(fn(self.v.data_ptr(), self.v_scale.data_ptr(), self.v_zp.data_ptr(), rows, d, vd.data_ptr(), d, stream))
        return kd.view(b, h, length, d)[:, :, :T], vd.view(b, h, length, d)[:, :, :T]

    def _prefill_step(self, query, key, value):
        """keys_values/kvcache/attn_weights.py:817-869 and keys_values/kvcache/base.py:567-581: fill the
        first slots, positions = arange, scores = 0, plain causal attention on the chunk, no weights."""
        b, hq, num, d = query.shape
        if not (0 < b <= self.max_batch_size):
            raise ValueError(f"batch size {b} must be in (0, {self.max_batch_size}]")
        if num > self.max_prefill_length:
            raise ValueError(f"prefill length {num} exceeds cache_length {self.cache_length}")
        self.batch_size = b
        index = torch.arange(num, dtype=torch.int32, device=self.device).view(1, 1, -1).expand(b, self.n_query_groups, -1).contiguous()
        self.scores.zero_()
        for extra in (self.v_norm, self.q_errors):
            if extra is not None:
                extra.zero_()
        self.current_length = num
        self._write(index, key, value, 0)
        if self.blocks_over_heads:
            self._block_errors(index, None, key, value)
            self._write_back(index, None, (0, num))
        if self.grace_period > 0:  # first slot to move out once the cache is full, attn_weights.py:861-863
            self.next_grace_pos = self.cache_length - self.grace_period
        self.prefill_length = num
        self._use_initial_rule = num == self.cache_length
        self._have_next = False
        self._input_pos = num
        out, _, _ = ops.prefill_core(query, key.to(self.dtype), value.to(self.dtype), self.scale_factor, 0, None,
                                     return_weights=False, output_transposed=True)
        return out.reshape(b, num, hq * d)

    def _write(self, index: torch.Tensor, key: torch.Tensor, value: torch.Tensor, input_pos: int):
        b, h, num = index.shape
        key = key.to(self.dtype)
        value = value.to(self.dtype)
        if key.stride(-1) != 1:
            key = key.contiguous()
        if value.stride(-1) != 1:
            value = value.contiguous()
        a = _lib.CacheWriteArgs()
        a.B, a.Hkv, a.num, a.D, a.cache_len = b, h, num, self.head_size, self.cache_length
        a.input_pos = input_pos
        codes = self.quantized and not self.blocks_over_heads
        a.kv_dtype = _lib.quant_kv_dtype(self.num_bits, self.dtype) if codes else _lib.elem_kv_dtype(self.dtype)
        a.index = index.data_ptr()
        a.index_stride_b, a.index_stride_h = index.stride(0), index.stride(1)
        a.key = key.data_ptr()
        a.key_stride_b, a.key_stride_h, a.key_stride_t = key.stride(0), key.stride(1), key.stride(2)
        a.value = value.data_ptr()
        a.value_stride_b, a.value_stride_h, a.value_stride_t = value.stride(0), value.stride(1), value.stride(2)
        a.k_cache = self.k.data_ptr()
        a.kc_stride_b, a.kc_stride_h, a.kc_stride_t = self.k.stride(0), self.k.stride(1), self.k.stride(2)
        a.v_cache = self.v.data_ptr()
        a.vc_stride_b, a.vc_stride_h, a.vc_stride_t = self.v.stride(0), self.v.stride(1), self.v.stride(2)
        if codes:
            a.k_scale, a.k_zp = self.k_scale.data_ptr(), self.k_zp.data_ptr()
            a.v_scale, a.v_zp = self.v_scale.data_ptr(), self.v_zp.data_ptr()
            a.qs_stride_b, a.qs_stride_h = self.k_scale.stride(0), self.k_scale.stride(1)
        a.token_pos = self.token_pos.data_ptr()
        a.tp_stride_b, a.tp_stride_h = self.token_pos.stride(0), self.token_pos.stride(1)
        a.scores = self.scores.data_ptr()
        a.sc_stride_b, a.sc_stride_h = self.scores.stride(0), self.scores.stride(1)
        # blocks over the heads: the row-quantising write cannot give the blocks' errors (_block_errors does)
        a.v_norm, a.q_errors = _lib.ptr(self.v_norm), (None if self.blocks_over_heads else _lib.ptr(self.q_errors))
        if self._log_on and self._log_arena is not None and input_pos >= self.cache_length:
            # keys_values/kvcache/attn_weights.py:629-633: the slots are recorded by the kernel that consumes them
            log_pos = input_pos - self.cache_length
            self._log_arena.reserve(log_pos + num)
            arena = self._log_arena.data
            a.replay_log, a.log_blocksize, a.log_pos = arena.data_ptr(), self.replay_log_blocksize, log_pos
            a.log_stride_block, a.log_stride_b, a.log_stride_h = arena.stride(0), arena.stride(1), arena.stride(2)
        ring = None
        if self.grace_period > 0 and input_pos >= self.cache_length:
            # keys_values/kvcache/attn_weights.py:267-303: the num2 oldest ring slots move out to
            # `index` and take the last num2 new tokens; wrap-around run starting at next_grace_pos
            gp = self.grace_period
            prefix = self.cache_length - gp
            num2 = min(num, gp)
            start = self.next_grace_pos - prefix
            ring = self._ring_twice[start : start + num2]
            a.grace_num, a.grace_period, a.grace_slots = num2, gp, ring.data_ptr()
            if num <= gp:  # attn_weights.py:601-606
                self.next_grace_pos = (self.next_grace_pos - prefix + num) % gp + prefix
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().kvx_cache_write(ctypes.byref(a), _lib.stream_ptr(self.device)))
        return ring

    def _h2o_args(self, full: bool, k: int = 1) -> _lib.H2OArgs:
        a = _lib.H2OArgs()
        a.B, a.Hkv, a.kv_len = self.batch_size, self.n_query_groups, self.current_length
        a.limit = self.cache_length - self.grace_period if full else self.current_length
        a.k = k if full else 1
        a.normalize = int(self.normalize_scores and full)
        a.input_pos = self._input_pos
        a.prefill_len = self.prefill_length
        a.scores = self.scores.data_ptr()
        a.sc_stride_b, a.sc_stride_h = self.scores.stride(0), self.scores.stride(1)
        a.token_pos = self.token_pos.data_ptr()
        a.tp_stride_b, a.tp_stride_h = self.token_pos.stride(0), self.token_pos.stride(1)
        a.v_norm = _lib.ptr(self.v_norm)
        a.q_errors = _lib.ptr(self.q_errors) if full else None  # only the selection reads them
        a.combination = self.combination_constant
        return a

    def _decode_h2o_step(self, query, kc, vc, quant) -> torch.Tensor:
        """``self.mha(...)`` and ``self._update(...)`` of keys_values/kvcache/base.py:583-595 for one new
        token and a full cache, as the single fused call ``kvx_sdpa_decode_h2o`` (selection size 1)."""
        if self.v_length or self.q_hitter:
            out, w, _ = ops.decode_core(query, kc, vc, self.scale_factor, return_weights=True, quant=quant)
            self._update(w, 1, select=1)
            return out
        # the lowest-score slot only: a following single-token step needs no more, anything longer selects again
        launch, out = self._decode_h2o_prepare(query, kc, vc, quant)
        launch()
        self._have_next = True
        self._next_count = 1
        return out

    def _decode_h2o_prepare(self, query, kc, vc, quant):
        """Argument blocks and workspace of one ``kvx_sdpa_decode_h2o`` call; returns the launcher (it
        may be called repeatedly: every call is one more update of the scores) and the output."""
        b, hq, _, d = query.shape
        dev = self.device
        lib = _lib.load()
        with torch.cuda.device(dev):
            out = torch.empty((b, hq, d), dtype=query.dtype, device=dev)
            o_view = out.unsqueeze(2)
            a = _lib.SdpaArgs()
            ops._fill_common(a, query, kc, vc, self.scale_factor, self.current_length - 1, None, quant, 0)
            a.o = o_view.data_ptr()
            a.o_stride_b, a.o_stride_h, a.o_stride_t = o_view.stride(0), o_view.stride(1), o_view.stride(2)
            h = self._h2o_args(True, 1)
            h.next_index = self._next_flat.data_ptr()
            nb_a = lib.kvx_sdpa_decode_h2o_workspace_bytes(ctypes.byref(a))
            nb_h = (lib.kvx_h2o_workspace_bytes(ctypes.byref(h)) + 255) // 256 * 256
            ws = _lib.workspace(dev, nb_a + nb_h)
            h.workspace, h.workspace_bytes = ws.data_ptr(), nb_h
            a.workspace, a.workspace_bytes = ws.data_ptr() + nb_h, ws.numel() - nb_h
            stream = _lib.stream_ptr(dev)

        def launch():
            with torch.cuda.device(dev):
                _lib.check(lib.kvx_sdpa_decode_h2o(ctypes.byref(a), ctypes.byref(h), stream))

        launch.keepalive = (query, kc, vc, quant, out, ws)
        return launch, out

    def _update(self, attn_weights: torch.Tensor, query_length: int, select: Optional[int] = None):
        """keys_values/kvcache/attn_weights.py:721-783 with keys_values/kvcache/h2o.py:146-199. ``select``: how
        many slots to choose now (default: as many as a next step may take, at most EAGER_SELECT)."""
        if not isinstance(attn_weights, torch.Tensor):
            raise TypeError("attn_weights argument needs to be torch.Tensor")
        if not isinstance(query_length, int) or query_length <= 0:
            raise TypeError("query_length argument needs to be positive int")
        shape = (self.batch_size, self.n_query_groups, self.current_length)
        if tuple(attn_weights.shape) != shape:
            raise ValueError(f"Shape of attn_weights must be {shape}, but attn_weights.shape = {tuple(attn_weights.shape)}")
        if attn_weights.dtype != torch.float32:
            raise ValueError(f"attn_weights.dtype={attn_weights.dtype}, must be {torch.float32}")
        _lib.require_gpu(attn_weights)
        attn_weights = attn_weights.contiguous()
        full = self.current_length == self.cache_length
        k_now = min(self._select_k, EAGER_SELECT) if select is None else min(select, self._select_k)
        a = self._h2o_args(full, k_now)
        a.w = attn_weights.data_ptr()
        a.q_len = query_length
        lib = _lib.load()
        with torch.cuda.device(self.device):
            if full:
                nxt = self._next_flat
            else:  # only the accumulation matters while slots are free; the choice is discarded
                nxt = torch.empty((self.batch_size, self.n_query_groups, 1), dtype=torch.int32, device=self.device)
            a.next_index = nxt.data_ptr()
            nbytes = lib.kvx_h2o_workspace_bytes(ctypes.byref(a))
            if not self._overlap:
                ws = _lib.workspace(self.device, nbytes)
                a.workspace = _lib.ptr(ws)
                a.workspace_bytes = 0 if ws is None else ws.numel()
                _lib.check(lib.kvx_h2o_update_select(ctypes.byref(a), _lib.stream_ptr(self.device)))
            else:
                main = torch.cuda.current_stream(self.device)
                self._second_stream()
                ready = torch.cuda.Event()
                ready.record(main)
                with torch.cuda.stream(self._side_stream):
                    self._side_stream.wait_event(ready)
                    ws = _lib.workspace(self.device, nbytes)  # one buffer per stream
                    a.workspace = _lib.ptr(ws)
                    a.workspace_bytes = 0 if ws is None else ws.numel()
                    _lib.check(lib.kvx_h2o_update_select(ctypes.byref(a), self._side_stream.cuda_stream))
                    done = torch.cuda.Event()
                    done.record(self._side_stream)
                self._select_done = done
                # the second stream reads these: tell the allocator, and keep them until the wait
                attn_weights.record_stream(self._side_stream)
                nxt.record_stream(self._side_stream)
                self._select_keep = (attn_weights, nxt)
        self._have_next = full
        self._next_count = k_now if full else 0


class VLengthH2OKVCache(H2OKVCache):
    """keys_values/kvcache/h2o.py:344-420: the instantaneous score is the attention weight times the
    norm of the slot's V row, normalised to sum to the number of queries."""

    def __init__(self, params: KVCacheParams, **kwargs):
        kwargs.pop("v_length", None)  # comes back through clone()
        super().__init__(params, v_length=True, **kwargs)


class QuantizedH2OKVCache(H2OKVCache):
    """keys_values/kvcache/qh2o.py:31-230: H2O scores and quantisation errors, both min-max
    normalised per batch element, in a convex combination. Quantised store only."""

    def __init__(self, params: KVCacheParams, **kwargs):
        kwargs.setdefault("quantized", True)
        kwargs.pop("q_hitter", None)  # comes back through clone()
        super().__init__(params, q_hitter=True, **kwargs)


class QuantizedVLengthH2OKVCache(H2OKVCache):
    """keys_values/kvcache/qh2o.py:233-330."""

    def __init__(self, params: KVCacheParams, **kwargs):
        kwargs.setdefault("quantized", True)
        kwargs.pop("q_hitter", None)  # come back through clone()
        kwargs.pop("v_length", None)
        super().__init__(params, q_hitter=True, v_length=True, **kwargs)


_CACHE_TYPES = {"h2o": H2OKVCache, "h2o-vlen": VLengthH2OKVCache, "qh2o": QuantizedH2OKVCache, "qh2o-vlen": QuantizedVLengthH2OKVCache}
_STORES = {"default": (False, 8), "torch-quantized8": (True, 8), "torch-quantized4": (True, 4)}


def create_kv_cache(name: str, params: KVCacheParams, **kwargs) -> H2OKVCache:
    """``<policy>-<store>`` as in keys_values/kvcache/factory.py:50-66 (``h2o-default``,
    ``h2o-vlen-torch-quantized8``, ``qh2o-torch-quantized8`` ...). Policies other than the H2O family
    and stores other than bf16 / 8-bit raise."""
    for store, (quantized, num_bits) in _STORES.items():
        if name.endswith("-" + store):
            policy = name[: -len(store) - 1]
            if policy not in _CACHE_TYPES:
                raise NotImplementedError(f"cache policy '{policy}' is not implemented; have {sorted(_CACHE_TYPES)}")
            return _CACHE_TYPES[policy](params, quantized=quantized, num_bits=num_bits, **kwargs)
    raise NotImplementedError(f"cache name '{name}': store must be one of {sorted(_STORES)}")
