"""
Replay log of an attention-weights cache: the token chunks it was fed and, for every token position
from ``cache_length`` on, the slot its K/V went to — what the reference records for gradient
computation and for recreating cache content (keys_values/kvcache/base.py:715-855,
keys_values/kvcache/attn_weights.py:43-204).

``AttnWeightsReplayLog`` has the reference's surface: ``token_chunks``, ``slot_positions`` (blocks of
shape ``(batch_size, n_query_groups, blocksize)``, uint32, the last one cut to the positions in use by
``finalize``), ``extract_index``, ``len()``. The live log inside a cache is a ``ReplayArena``: all blocks
in ONE device allocation ``(blocks, batch, heads, blocksize)`` that ``kvx_cache_write`` fills as it
consumes the slots (no extra launch, no per-block allocation); the blocks handed out are views of it.
"""
from typing import List, Optional, Tuple

import torch

DEFAULT_REPLAY_LOG_BLOCKSIZE = 1024  # keys_values/kvcache/attn_weights.py:319


class AttnWeightsReplayLog:
    def __init__(
        self,
        token_chunks: List[torch.Tensor],
        slot_positions: List[torch.Tensor],
        cache_length: int,
        max_prefill_length: int,
        blocksize: int,
        grace_period: int = 0,
    ):
        if token_chunks:
            device = token_chunks[0].device
            if any(c.device != device for c in token_chunks):
                raise ValueError("All token_chunks entries must be on same device")
        if slot_positions:
            if not token_chunks:
                raise ValueError("Cannot have empty token_chunks, non-empty slot_positions")
            shape = slot_positions[0].shape[:-1]
            if not all(b.shape[:-1] == shape for b in slot_positions):
                raise ValueError("Blocks in slot_positions have incompatible shapes")
            if any(c.shape[0] != shape[0] for c in token_chunks):
                raise ValueError(f"slot_positions has batch size {shape[0]}, but some token_chunks entries differ")
        self._token_chunks = token_chunks
        self._slot_positions = slot_positions
        self._cache_length = cache_length
        self._max_prefill_length = max_prefill_length
        self._grace_period = grace_period
        self.blocksize = blocksize

    @property
    def token_chunks(self) -> List[torch.Tensor]:
        return self._token_chunks

    @property
    def slot_positions(self) -> List[torch.Tensor]:
        return self._slot_positions

    @property
    def cache_length(self) -> int:
        return self._cache_length

    @property
    def max_prefill_length(self) -> int:
        return self._max_prefill_length

    @property
    def grace_period(self) -> int:
        return self._grace_period

    @property
    def device(self) -> Optional[torch.device]:
        if self._slot_positions:
            return self._slot_positions[0].device
        return self._token_chunks[0].device if self._token_chunks else None

    def __len__(self) -> int:
        """Length of the token sequence (keys_values/kvcache/base.py:734-740)."""
        return sum(chunk.shape[-1] for chunk in self._token_chunks)

    def _position_and_offset(self, input_pos: int) -> Tuple[int, int]:
        """keys_values/kvcache/attn_weights.py:153-172."""
        if input_pos < self.cache_length:
            raise ValueError(f"token_pos = {input_pos} must be >= {self.cache_length} = cache_length")
        pos = self.cache_length
        for relpos, block in enumerate(self._slot_positions):
            if input_pos < pos + block.shape[-1]:
                return relpos, input_pos - pos
            pos += block.shape[-1]
        raise ValueError(f"token_pos = {input_pos} is too large")

    def extract_index(self, input_pos: int, num: int, dtype: Optional[torch.dtype] = None,
                      device: Optional[torch.device] = None) -> torch.Tensor:
        """Slots that token positions ``input_pos .. input_pos + num - 1`` were written to,
        ``(batch_size, n_query_groups, num)`` (keys_values/kvcache/attn_weights.py:174-204)."""
        relpos, bstart = self._position_and_offset(input_pos)
        if dtype is None:
            dtype = torch.int64
        if device is None:
            device = self.device
        parts = []
        done = 0
        while done < num:
            if relpos >= len(self._slot_positions):
                raise ValueError(f"token_pos = {input_pos + num - 1} is too large")
            block = self._slot_positions[relpos]
            bend = min(bstart + num - done, block.shape[-1])
            # uint32 -> int32 is a bit cast (slots are far below 2^31); conversions from int32 exist everywhere
            parts.append(block[:, :, bstart:bend].view(torch.int32).to(dtype=dtype, device=device))
            done += bend - bstart
            relpos += 1
            bstart = 0
        return torch.cat(parts, dim=-1)


class ReplayArena:
    """Growing store of slot-position blocks, ``(blocks, batch, heads, blocksize)`` int32 on the device
    (the bits of the reference's uint32 blocks)."""

    def __init__(self, batch_size: int, n_query_groups: int, blocksize: int, device: torch.device):
        self.shape = (batch_size, n_query_groups, blocksize)
        self.blocksize = blocksize
        self.device = device
        self.data = torch.zeros((4,) + self.shape, dtype=torch.int32, device=device)  # new blocks start at 0, attn_weights.py:147-151

    def reserve(self, positions: int):
        """Make room for log positions ``0 .. positions - 1``."""
        need = (positions + self.blocksize - 1) // self.blocksize
        have = self.data.shape[0]
        if need > have:
            grown = torch.zeros((max(need, 2 * have),) + self.shape, dtype=torch.int32, device=self.device)
            grown[:have] = self.data
            self.data = grown

    def blocks(self, positions: int) -> List[torch.Tensor]:
        """The blocks covering log positions ``0 .. positions - 1`` as uint32 views, the last one cut
        to the positions in use (keys_values/kvcache/attn_weights.py:102-123)."""
        out = []
        for i in range((positions + self.blocksize - 1) // self.blocksize):
            used = min(self.blocksize, positions - i * self.blocksize)
            out.append(self.data[i, :, :, :used].view(torch.uint32))
        return out
