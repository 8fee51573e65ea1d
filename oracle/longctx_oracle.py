"""
CPU oracle for the callers of the attention / cache path (normalisation, rotary encoding, the
Qwen3-shaped block and the chunked prefill loop).  TEST INFRASTRUCTURE ONLY: imported by tests and by
the ``cpu_baseline`` leg of the benchmark, never by the library.

Each function cites the reference lines it restates (paths relative to the reference root). Pinning
(tests/test_longctx.py): ``rmsnorm`` against the closed form on constant and one-hot rows and against
a float64 evaluation; the rotary encoding against its invariants (it preserves the norm of every
(d, d + D/2) pair, position 0 is the identity, and q.k after rotation depends on the position
difference only) and against the explicit per-pair 2x2 rotation; the chunk schedule against the
properties its reference asserts (keys_values/long_context.py:123-160: sizes add up, the first chunk is
the prefill length, no cache length inside a chunk) and the reference's cursor walk on random cases;
``qk_norm_rope`` row by row against the pinned pieces (which head gets which weight, each token its own
position, values untouched) and against scalar arithmetic with both bf16 roundings written out;
``PrefillOracle`` by zero output projections (the stack must reduce to the final norm of the
embeddings) and by one block on tiny widths recomputed token by token with explicit matrix-vector
products, the pinned row functions and a cache oracle of its own. The MLP is litgpt's LLaMAMLP
(``proj(silu(fc_1 x) * fc_2 x)``); litgpt is not part of the reference tree (unpinned dependency of
it), so that formula is restated from its published source: parity unpinned.
"""
import math
from typing import List, Optional

import torch
import torch.nn.functional as F

from oracle import kvx_oracle as O


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm.forward, keys_values/model.py:870-878 (dim = -1, no unit offset)."""
    dtype = x.dtype
    x32 = x.to(torch.float32)
    norm_x = torch.linalg.vector_norm(x32, dim=-1, keepdim=True) * (1.0 / math.sqrt(x.shape[-1]))
    x32 = x32 / (norm_x + eps)
    return (x32 * weight).to(dtype)


def rope_tables(context: int, head_size: int, base: float):
    inv = 1.0 / (base ** (torch.arange(0, head_size, 2, dtype=torch.float32) / head_size))
    ang = torch.arange(context, dtype=torch.float32).unsqueeze(-1) * inv
    return ang.cos(), ang.sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x (..., T, D), cos / sin (T, D/2): y = x * cos + cat(-x2, x1) * sin in fp32, cast back
    (keys_values/pos_encoding.py:34-44 with the half-split convention of
    keys_values/fused/fused_rope.py:57-87,198-200)."""
    D = x.shape[-1]
    c = torch.cat((cos, cos), dim=-1)
    s = torch.cat((sin, sin), dim=-1)
    x32 = x.to(torch.float32)
    x1, x2 = x32[..., : D // 2], x32[..., D // 2 :]
    return (x32 * c + torch.cat((-x2, x1), dim=-1) * s).to(x.dtype)


def qk_norm_rope(qkv, n_head, n_query_groups, head_size, q_weight, k_weight, eps, cos, sin, input_pos):
    """keys_values/model.py:686-775: split, view, transpose, norm_q / norm_k, rotary encoding.
    qkv (B, num, (n_head + 2 n_query_groups) * head_size). Returns q (B, n_head, num, hs), k, v."""
    B, num, _ = qkv.shape
    qs, ks = n_head * head_size, n_query_groups * head_size
    q, k, v = qkv.split((qs, ks, ks), dim=-1)
    q = q.view(B, num, n_head, head_size).transpose(1, 2)
    k = k.view(B, num, n_query_groups, head_size).transpose(1, 2)
    v = v.view(B, num, n_query_groups, head_size).transpose(1, 2)
    if q_weight is not None:
        q = rmsnorm(q, q_weight, eps)
        k = rmsnorm(k, k_weight, eps)
    c, s = cos[input_pos : input_pos + num], sin[input_pos : input_pos + num]
    return apply_rope(q, c, s), apply_rope(k, c, s), v


class PrefillOracle:
    """The chunked prefill of keys_values_amd.longctx.model restated on the CPU with the cache oracle
    (block: keys_values/model.py:524-584; loop: keys_values/long_context.py:601-662). ``weights`` is a
    list of per-layer dicts (qkv, proj, fc_1, fc_2, mlp_proj, norm_1, norm_2, norm_q, norm_k)."""

    def __init__(self, cfg, wte, weights: List[dict], ln_f, cache_length: int, chunk_size: int, batch_size: int, quantized: bool,
                 max_context: int):
        self.cfg, self.wte, self.weights, self.ln_f = cfg, wte, weights, ln_f
        self.quantized = quantized
        self.caches = [O.H2OCacheOracle(batch_size, cfg.n_head, cfg.n_query_groups, cache_length, cfg.head_size, dtype=torch.bfloat16,
                                        max_chunk_size=chunk_size) for _ in weights]
        self.cos, self.sin = rope_tables(max_context, cfg.head_size, cfg.rope_base)
        self.input_pos = 0

    def _stored(self, x):
        return O.dequantize_rows(*O.quantize_rows(x)) if self.quantized else x

    def forward_chunk(self, input_ids: torch.Tensor, forced_index: Optional[list] = None):
        cfg = self.cfg
        x = F.embedding(input_ids, self.wte)
        B, num, _ = x.shape
        for li, w in enumerate(self.weights):
            xn = rmsnorm(x, w["norm_1"], cfg.norm_eps)
            qkv = F.linear(xn, w["qkv"])
            q, k, v = qk_norm_rope(qkv, cfg.n_head, cfg.n_query_groups, cfg.head_size, w["norm_q"], w["norm_k"], cfg.norm_eps,
                                   self.cos, self.sin, self.input_pos)
            cache = self.caches[li]
            if cache.input_pos == 0:
                o = cache.prefill(q, k, v, self._stored(k), self._stored(v))
            else:
                if forced_index is not None and forced_index[li] is not None:
                    cache.next_index = forced_index[li]
                o, _, _ = cache.forward(q, self._stored(k), self._stored(v))
            y = o.transpose(1, 2).reshape(B, num, cfg.n_head * cfg.head_size)
            x = x + F.linear(y, w["proj"])
            xn = rmsnorm(x, w["norm_2"], cfg.norm_eps)
            h = F.silu(F.linear(xn, w["fc_1"])) * F.linear(xn, w["fc_2"])
            x = x + F.linear(h, w["mlp_proj"])
        self.input_pos += num
        return rmsnorm(x, self.ln_f, cfg.norm_eps)
