"""Chunk schedule of the long-context forward pass.

Contract (``create_chunk_sizes`` with ``randomize_chunk_sizes=False``, keys_values/long_context.py:45-121,
checked there by ``_assert_chunk_sizes``, :123-160):

* the first chunk is the prefill: the smallest ``max_prefill_length`` of the caches;
* every cache length that the sequence reaches is the end of a chunk, so that a cache is never filled
  up in the middle of a chunk;
* between two such cuts the tokens go in chunks of ``chunk_size``; what is left before a cut makes one
  more chunk, unless it is ``ABSORB`` tokens or fewer, in which case the chunk before it takes them;
* behind the last cut: chunks of ``chunk_size`` and one remainder.
"""
from typing import List, Sequence

ABSORB = 4  # a chunk that would end this close to a cut ends on it (CLOSEBY_THRESHOLD, keys_values/long_context.py:40)


def _cover(span: int, chunk_size: int, ends_on_cut: bool) -> List[int]:
    """Chunk sizes for ``span`` tokens that start on a chunk boundary."""
    if span <= 0:
        return []
    if not ends_on_cut:
        whole, rest = divmod(span, chunk_size)
        return [chunk_size] * whole + ([rest] if rest else [])
    # whole chunks as long as more than chunk_size + ABSORB tokens remain; the last chunk takes the rest
    whole = max(0, -((chunk_size + ABSORB - span) // chunk_size))
    return [chunk_size] * whole + [span - whole * chunk_size]


def create_chunk_sizes(max_prefill_length: int, cache_lengths: Sequence[int], seq_length: int, chunk_size: int) -> List[int]:
    """``max_prefill_length``: minimum over the caches; ``cache_lengths``: the caches' lengths.
    Returns the chunk sizes, which add up to ``seq_length``."""
    if seq_length <= 0 or chunk_size <= 0 or max_prefill_length <= 0:
        raise ValueError("seq_length, chunk_size and max_prefill_length must be positive")
    reached = sorted({int(c) for c in cache_lengths if c <= seq_length})
    if not reached:
        # no cache fills up: the prefill and, if the sequence is longer, all the rest in one chunk
        # (keys_values/long_context.py:81-86)
        first = min(max_prefill_length, seq_length)
        return [first] + ([seq_length - first] if seq_length > first else [])
    if reached[0] < max_prefill_length:
        raise ValueError(f"cache length {reached[0]} is below the prefill length {max_prefill_length}")
    sizes = [max_prefill_length]
    at = max_prefill_length
    for cut in reached:
        sizes += _cover(cut - at, chunk_size, ends_on_cut=True)
        at = cut
    sizes += _cover(seq_length - at, chunk_size, ends_on_cut=False)
    assert sum(sizes) == seq_length
    return sizes
