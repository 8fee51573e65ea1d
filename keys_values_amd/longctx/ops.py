"""Host wrappers of the normalisation / rotary / gated-activation kernels (C ABI: kvx_rmsnorm_rows,
kvx_add_rmsnorm_rows, kvx_swiglu_rows, kvx_qk_norm_rope)."""
from typing import Optional, Tuple

import torch

from keys_values_amd import _lib


def rope_tables(context: int, head_size: int, base: float, device) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 cos / sin tables (context, head_size / 2): row p holds cos / sin of p * base^(-2j / head_size).
    Half-split convention: element d of a head is paired with d +- head_size / 2
    (keys_values/fused/fused_rope.py:57-87,198-200)."""
    inv = 1.0 / (base ** (torch.arange(0, head_size, 2, dtype=torch.float32, device=device) / head_size))
    ang = torch.arange(context, dtype=torch.float32, device=device).unsqueeze(-1) * inv
    return ang.cos().contiguous(), ang.sin().contiguous()


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm.forward over the last axis (keys_values/model.py:870-878). x bf16 (..., dim), rows contiguous."""
    _lib.require_gpu(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.float32:
        raise ValueError("rmsnorm takes bfloat16 rows and a float32 weight")
    dim = x.shape[-1]
    if weight.shape != (dim,):
        raise ValueError(f"weight.shape = {tuple(weight.shape)}, must be ({dim},)")
    x2 = x.reshape(-1, dim)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    o2 = out.view(-1, dim)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.kvx_rmsnorm_rows(x2.data_ptr(), x2.stride(0), o2.data_ptr(), o2.stride(0), weight.data_ptr(), x2.shape[0], dim,
                                        float(eps), _lib.stream_ptr(x.device)))
    return out


def add_rmsnorm_(x: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x += delta`` (in place, rounded to bf16) and ``RMSNorm(x)`` in one pass: the residual add of a
    block with the normalisation that follows it (keys_values/model.py:560-584). Returns the normed rows."""
    _lib.require_gpu(x, delta, weight)
    if x.dtype != torch.bfloat16 or delta.dtype != torch.bfloat16 or weight.dtype != torch.float32:
        raise ValueError("add_rmsnorm_ takes bfloat16 rows and a float32 weight")
    dim = x.shape[-1]
    if x.shape != delta.shape or weight.shape != (dim,) or not x.is_contiguous():
        raise ValueError(f"x {tuple(x.shape)} (contiguous), delta {tuple(delta.shape)}, weight {tuple(weight.shape)} do not fit")
    d2 = delta.reshape(-1, dim)
    if d2.stride(-1) != 1:
        d2 = d2.contiguous()
    x2 = x.view(-1, dim)
    out = torch.empty_like(x)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        _lib.check(lib.kvx_add_rmsnorm_rows(x2.data_ptr(), dim, d2.data_ptr(), d2.stride(0), x2.data_ptr(), dim, out.data_ptr(), dim,
                                            weight.data_ptr(), x2.shape[0], dim, float(eps), _lib.stream_ptr(x.device)))
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` for ``gate_up = [gate | up]`` (..., 2 * dim), the output of one GEMM over the
    stacked fc_1 / fc_2 weights; same rounding as ``F.silu(gate) * up`` on bf16 tensors."""
    _lib.require_gpu(gate_up)
    if gate_up.dtype != torch.bfloat16 or gate_up.shape[-1] % 16 != 0:
        raise ValueError("swiglu takes bfloat16 rows of even width, a multiple of 16")
    dim = gate_up.shape[-1] // 2
    g2 = gate_up.reshape(-1, 2 * dim)
    if g2.stride(-1) != 1:
        g2 = g2.contiguous()
    out = torch.empty(gate_up.shape[:-1] + (dim,), dtype=gate_up.dtype, device=gate_up.device)
    lib = _lib.load()
    with torch.cuda.device(gate_up.device):
        _lib.check(lib.kvx_swiglu_rows(g2.data_ptr(), g2.stride(0), out.data_ptr(), dim, g2.shape[0], dim, _lib.stream_ptr(gate_up.device)))
    return out


def qk_norm_rope_(qkv: torch.Tensor, n_head: int, n_query_groups: int, head_size: int, q_weight: Optional[torch.Tensor],
                  k_weight: Optional[torch.Tensor], eps: float, cos: torch.Tensor, sin: torch.Tensor, input_pos: int) -> torch.Tensor:
    """In place on qkv (B, num, (n_head + 2 n_query_groups) * head_size): norm_q / norm_k over each
    head and the rotary encoding at positions input_pos .. input_pos + num - 1
    (keys_values/model.py:733-775). Returns qkv."""
    _lib.require_gpu(qkv, cos, sin)
    if qkv.dtype != torch.bfloat16 or qkv.ndim != 3 or qkv.stride(-1) != 1:
        raise ValueError("qkv must be a bfloat16 (B, num, heads * head_size) tensor with a contiguous last axis")
    B, num, width = qkv.shape
    if width != (n_head + 2 * n_query_groups) * head_size:
        raise ValueError(f"qkv.shape[-1] = {width} does not fit {n_head} + 2 * {n_query_groups} heads of {head_size}")
    if cos.shape != sin.shape or cos.ndim != 2 or cos.shape[1] != head_size // 2 or cos.dtype != torch.float32:
        raise ValueError("cos / sin must be float32 (positions, head_size / 2) tables")
    lib = _lib.load()
    with torch.cuda.device(qkv.device):
        _lib.check(lib.kvx_qk_norm_rope(qkv.data_ptr(), qkv.stride(0), qkv.stride(1), B, num, n_head, n_query_groups, head_size,
                                        _lib.ptr(q_weight), _lib.ptr(k_weight), float(eps), cos.data_ptr(), sin.data_ptr(),
                                        cos.shape[0], int(input_pos), _lib.stream_ptr(qkv.device)))
    return qkv
