"""Chunk schedule of the long-context forward pass."""
from typing import List, Sequence

CLOSEBY_THRESHOLD = 4  # keys_values/long_context.py:40


def create_chunk_sizes(max_prefill_length: int, cache_lengths: Sequence[int], seq_length: int, chunk_size: int) -> List[int]:
    """Deterministic branch (``randomize_chunk_sizes=False``) of ``create_chunk_sizes``,
    keys_values/long_context.py:45-121: the first chunk has the smallest ``max_prefill_length`` of
    the caches, later chunks have ``chunk_size`` tokens, and no cache length falls inside a chunk (a
    chunk that would end within ``CLOSEBY_THRESHOLD`` tokens of one, or beyond it, ends exactly there).

    ``max_prefill_length``: min over the caches; ``cache_lengths``: the caches' lengths."""
    if seq_length <= 0 or chunk_size <= 0 or max_prefill_length <= 0:
        raise ValueError("seq_length, chunk_size and max_prefill_length must be positive")
    mpl = max_prefill_length
    points_to_cover = sorted(set(c for c in cache_lengths if c <= seq_length))
    if not points_to_cover:
        return [seq_length] if mpl >= seq_length else [mpl, seq_length - mpl]
    chunk_sizes = [mpl]
    num_done = mpl
    while num_done < seq_length:
        c_size = min(chunk_size, seq_length - num_done)
        next_pt = num_done + c_size
        if points_to_cover and next_pt >= points_to_cover[0] - CLOSEBY_THRESHOLD:
            c_size = points_to_cover.pop(0) - num_done
        if c_size > 0:
            chunk_sizes.append(c_size)
        num_done += c_size
    if sum(chunk_sizes) != seq_length:
        raise AssertionError(f"chunk sizes {chunk_sizes} do not add up to {seq_length}")
    return chunk_sizes
