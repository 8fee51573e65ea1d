"""Shared input builders for the tests (seeded, CPU generators as the benchmark inputs are)."""
import torch


def randn(gen, *shape, dtype=torch.bfloat16):
    return torch.randn(*shape, generator=gen, dtype=torch.float32).to(dtype)


def make_qkv(seed, B, Hq, Hkv, q_len, T, D, dtype=torch.bfloat16):
    gen = torch.Generator().manual_seed(seed)
    q = randn(gen, B, Hq, q_len, D, dtype=dtype)
    k = randn(gen, B, Hkv, T, D, dtype=dtype)
    v = randn(gen, B, Hkv, T, D, dtype=dtype)
    return q, k, v, gen


def scattered_positions(gen, B, Hkv, T, input_pos, q_len):
    """Token positions of a cache after eviction-style writes: every (b, h) row holds the current
    chunk's positions input_pos .. input_pos+q_len-1 exactly once, in random slots, and distinct
    older positions (< input_pos) everywhere else (keys_values/attention/sdpa_wrapper.py:82-86)."""
    assert input_pos >= T - q_len
    tp = torch.empty(B, Hkv, T, dtype=torch.int32)
    for b in range(B):
        for h in range(Hkv):
            old = torch.randperm(input_pos, generator=gen)[: T - q_len].to(torch.int32)
            allp = torch.cat((old, torch.arange(input_pos, input_pos + q_len, dtype=torch.int32)))
            tp[b, h] = allp[torch.randperm(T, generator=gen)]
    return tp


def rel_err(a, b):
    a = a.double()
    b = b.double()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()
