"""
Qwen3-shaped decoder stack for chunked long-context prefill over H2O caches.

Follows the reference's inference path: ``LongContextInferenceModel.forward``
(keys_values/long_context.py:601-662) walks the prompt in chunks (schedule.create_chunk_sizes); each
chunk passes through every ``Block`` (keys_values/model.py:524-584, non-parallel residual) whose
attention writes to and reads from that layer's KV cache (keys_values/model.py:686-811,
keys_values/kvcache/base.py:554-595). Weights are random (normal, std 0.02, as
keys_values/model.py:294-301); the linear layers are plain library GEMMs through PyTorch, everything
else runs on the HIP kernels of this package. There is no CPU path.
"""
import os
from dataclasses import dataclass
from typing import List, Optional

import torch
import torch.nn.functional as F

from keys_values_amd import _lib
from keys_values_amd.kvcache.h2o import H2OKVCache, KVCacheParams
from keys_values_amd.longctx import ops
from keys_values_amd.longctx.schedule import create_chunk_sizes


@dataclass(frozen=True)
class PrefillConfig:
    n_layer: int
    n_embd: int
    n_head: int
    n_query_groups: int
    head_size: int
    intermediate_size: int
    vocab_size: int
    rope_base: float = 1.0e6
    norm_eps: float = 1.0e-6
    norm_qk: bool = True


# Qwen3-4B architecture numbers
QWEN3_4B = PrefillConfig(n_layer=36, n_embd=2560, n_head=32, n_query_groups=8, head_size=128, intermediate_size=9728, vocab_size=151936)


class _Layer:
    def __init__(self, cfg: PrefillConfig, gen: torch.Generator, device):
        def w(out_f, in_f):
            return (torch.randn((out_f, in_f), generator=gen, device=device, dtype=torch.float32) * 0.02).to(torch.bfloat16)

        d = cfg.head_size
        self.qkv = w((cfg.n_head + 2 * cfg.n_query_groups) * d, cfg.n_embd)
        self.proj = w(cfg.n_embd, cfg.n_head * d)
        # fc_1 and fc_2 stacked: one GEMM gives [gate | up] (the two halves are views of it)
        self.fc_12 = torch.cat((w(cfg.intermediate_size, cfg.n_embd), w(cfg.intermediate_size, cfg.n_embd)))
        self.fc_1, self.fc_2 = self.fc_12[: cfg.intermediate_size], self.fc_12[cfg.intermediate_size :]
        self.mlp_proj = w(cfg.n_embd, cfg.intermediate_size)
        self.norm_1 = torch.ones(cfg.n_embd, dtype=torch.float32, device=device)
        self.norm_2 = torch.ones(cfg.n_embd, dtype=torch.float32, device=device)
        self.norm_q = torch.ones(d, dtype=torch.float32, device=device) if cfg.norm_qk else None
        self.norm_k = torch.ones(d, dtype=torch.float32, device=device) if cfg.norm_qk else None


GEMM_TABLE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_table_gfx950.csv")


def use_gemm_table(path: str = GEMM_TABLE) -> bool:
    """Opt-in, process-wide: fix which library kernel serves each GEMM shape of this stack.

    The linear layers are plain library GEMMs, and which kernel serves a shape is the library's choice; its
    default is a poor one for some of the shapes of this stack. The table next to this file records, per shape
    (Qwen3-4B widths, chunks of 1024 and 16384 tokens), the kernel PyTorch's TunableOp measured as fastest on
    gfx950; it is read with tuning switched off, so nothing is measured at run time and the choice is the same in
    every run. This switches TunableOp on for EVERY GEMM of the process (shapes outside the table keep the
    library default, but the table's shapes change kernel, and with it summation order, wherever they occur),
    which is why nothing calls it implicitly. The file names the library versions it was made with: PyTorch
    refuses it under other versions; then, or on any other failure, the switches of TunableOp are put back as
    they were found and False is returned. TunableOp's own results file name is left alone."""
    import torch.cuda.tunable as tunable

    if not os.path.exists(path):
        return False
    try:
        before = (tunable.is_enabled(), tunable.tuning_is_enabled(), tunable.record_untuned_is_enabled())
    except Exception:  # a PyTorch without TunableOp
        return False
    ok = False
    try:
        tunable.enable(True)
        tunable.tuning_enable(False)
        tunable.record_untuned_enable(False)
        ok = bool(tunable.read_file(path))
    except Exception:  # a table it cannot parse
        ok = False
    if not ok:
        tunable.enable(before[0])
        tunable.tuning_enable(before[1])
        tunable.record_untuned_enable(before[2])
    return ok


class LongContextPrefillModel:
    def __init__(self, cfg: PrefillConfig, cache_length: int, chunk_size: int, max_batch_size: int = 1, quantized: bool = True,
                 max_context: int = 131072, seed: int = 4, device: Optional[torch.device] = None, gemm_table: bool = False):
        """``gemm_table=True`` calls :func:`use_gemm_table` (process-wide, see there); off by default."""
        self.cfg = cfg
        self.gemm_table = use_gemm_table() if gemm_table else False
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        if self.device.type != "cuda":
            raise RuntimeError("LongContextPrefillModel runs on a ROCm device only")
        if cfg.n_head % cfg.n_query_groups != 0:
            raise ValueError("n_head must be a multiple of n_query_groups")
        _lib.load()  # fail early if the kernels are not built
        gen = torch.Generator(device=self.device).manual_seed(seed)
        self.wte = (torch.randn((cfg.vocab_size, cfg.n_embd), generator=gen, device=self.device, dtype=torch.float32) * 0.02).to(torch.bfloat16)
        self.layers: List[_Layer] = [_Layer(cfg, gen, self.device) for _ in range(cfg.n_layer)]
        self.ln_f = torch.ones(cfg.n_embd, dtype=torch.float32, device=self.device)
        self.chunk_size = chunk_size
        self.cache_length = cache_length
        params = KVCacheParams(max_batch_size, cfg.n_query_groups, cache_length, cfg.head_size, cfg.n_head)
        # the eviction choice of a layer is first needed when the next chunk reaches that layer: it runs beside
        # the layer's dense part on a second stream
        self.caches = [H2OKVCache(params, max_chunk_size=chunk_size, quantized=quantized, device=self.device, overlap_select=True)
                       for _ in range(cfg.n_layer)]
        self.cos, self.sin = ops.rope_tables(max_context, cfg.head_size, cfg.rope_base, self.device)
        self.input_pos = 0

    def reset(self):
        """Start a new sequence (GPT.reset, keys_values/long_context.py:655): the next chunk is a prefill."""
        for c in self.caches:
            c._input_pos = 0
        self.input_pos = 0

    def chunk_sizes(self, seq_length: int) -> List[int]:
        mpl = min(c.max_prefill_length for c in self.caches)
        return create_chunk_sizes(mpl, [c.cache_length for c in self.caches], seq_length, self.chunk_size)

    def _block(self, li: int, x: torch.Tensor, xn: torch.Tensor, next_norm: torch.Tensor) -> torch.Tensor:
        """Block.forward, keys_values/model.py:524-584 (non-parallel residual, no post-norms). x is the
        residual stream (updated in place), xn = norm_1(x); returns the next block's norm_1 (or the final
        norm) of the updated stream: each residual add is fused with the normalisation that follows it."""
        cfg, layer = self.cfg, self.layers[li]
        B, num, _ = x.shape
        d, hq, hkv = cfg.head_size, cfg.n_head, cfg.n_query_groups
        qkv = F.linear(xn, layer.qkv)
        ops.qk_norm_rope_(qkv, hq, hkv, d, layer.norm_q, layer.norm_k, cfg.norm_eps, self.cos, self.sin, self.input_pos)
        q = qkv[..., : hq * d].view(B, num, hq, d).transpose(1, 2)
        k = qkv[..., hq * d : (hq + hkv) * d].view(B, num, hkv, d).transpose(1, 2)
        v = qkv[..., (hq + hkv) * d :].view(B, num, hkv, d).transpose(1, 2)
        y = self.caches[li].forward(q, k, v)
        xn = ops.add_rmsnorm_(x, F.linear(y, layer.proj), layer.norm_2, cfg.norm_eps)  # x = attention_output + x; norm_2(x)
        h = ops.swiglu(F.linear(xn, layer.fc_12))  # LLaMAMLP: proj(silu(fc_1 x) * fc_2 x)
        return ops.add_rmsnorm_(x, F.linear(h, layer.mlp_proj), next_norm, cfg.norm_eps)  # x = mlp_output + x

    def forward_chunk(self, input_ids: torch.Tensor) -> torch.Tensor:
        """One chunk through all layers; returns the final-norm hidden states (B, num, n_embd)."""
        if input_ids.ndim != 2:
            raise ValueError(f"input_ids.shape = {tuple(input_ids.shape)}, must be 2D")
        n = self.cfg.n_layer
        x = F.embedding(input_ids.to(self.device), self.wte)
        xn = ops.rmsnorm(x, self.layers[0].norm_1, self.cfg.norm_eps) if n > 0 else ops.rmsnorm(x, self.ln_f, self.cfg.norm_eps)
        for li in range(n):
            xn = self._block(li, x, xn, self.layers[li + 1].norm_1 if li + 1 < n else self.ln_f)
        self.input_pos += input_ids.shape[1]
        return xn

    def prefill(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Process whole sequences chunk by chunk; returns the hidden states of the last chunk."""
        self.reset()
        input_ids = input_ids.to(self.device)  # one copy: a copy per chunk from pageable memory would drain the stream every chunk
        out = None
        start = 0
        for n in self.chunk_sizes(input_ids.shape[1]):
            out = self.forward_chunk(input_ids[:, start : start + n])
            start += n
        return out
