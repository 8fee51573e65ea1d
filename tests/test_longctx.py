"""Callers of the path: chunk schedule, RMS normalisation, fused QK-norm + rotary kernel, and the
Qwen3-shaped chunked prefill against the CPU oracle."""
import math

import pytest
import torch

from keys_values_amd.longctx.schedule import create_chunk_sizes
from oracle import kvx_oracle as O
from oracle import longctx_oracle as LO


# ---- CPU: schedule and oracle pins ------------------------------------------------------------------


@pytest.mark.parametrize("mpl,lengths,seq,chunk", [(16384, [16384] * 36, 131072, 1024), (256, [256], 520, 64), (100, [100, 300], 1000, 64),
                                                   (512, [512], 300, 64), (64, [1 << 20], 1000, 128)])
def test_chunk_sizes_properties(mpl, lengths, seq, chunk):
    # what keys_values/long_context.py:123-160 (_assert_chunk_sizes) and the docstring of create_chunk_sizes demand
    sizes = create_chunk_sizes(mpl, lengths, seq, chunk)
    assert sum(sizes) == seq and all(s > 0 for s in sizes)
    assert sizes[0] == min(mpl, seq)
    ends = set()
    pos = 0
    for s in sizes:
        pos += s
        ends.add(pos)
    for length in lengths:
        if length <= seq:
            assert length in ends, f"cache length {length} falls inside a chunk of {sizes}"
    if any(length <= seq for length in lengths):  # otherwise the reference returns [prefill, rest] (long_context.py:81-86)
        assert all(s <= chunk + chunk // 2 or i == 0 for i, s in enumerate(sizes))
    else:
        assert sizes == ([seq] if mpl >= seq else [mpl, seq - mpl])


def test_chunk_sizes_config5():
    sizes = create_chunk_sizes(16384, [16384] * 36, 131072, 1024)
    assert sizes == [16384] + [1024] * 112


def test_rmsnorm_oracle_closed_forms():
    w = torch.linspace(0.5, 1.5, 64)
    # constant row c: |x|/sqrt(n) = |c|  ->  y = c / (|c| + eps) * w
    x = torch.full((3, 64), -2.0)
    torch.testing.assert_close(LO.rmsnorm(x, w, 1e-6), (-2.0 / (2.0 + 1e-6)) * w.expand(3, 64))
    # one-hot row a * e_j: norm = |a| / sqrt(n)
    x = torch.zeros(1, 64)
    x[0, 5] = 3.0
    y = LO.rmsnorm(x, w, 1e-2)
    assert y[0, 5].item() == pytest.approx(3.0 / (3.0 / 8.0 + 1e-2) * w[5].item(), rel=1e-6)
    assert y.abs().sum().item() == pytest.approx(abs(y[0, 5].item()))
    # float64 evaluation of the formula; eps is added to the norm, NOT to the mean square
    x = torch.randn(7, 96, generator=torch.Generator().manual_seed(0))
    x64 = x.double()
    ref = x64 / (x64.norm(dim=-1, keepdim=True) / math.sqrt(96) + 0.1) * torch.ones(96, dtype=torch.float64)
    torch.testing.assert_close(LO.rmsnorm(x, torch.ones(96), 0.1).double(), ref, rtol=1e-5, atol=1e-6)
    wrong = x64 / torch.sqrt((x64 * x64).mean(-1, keepdim=True) + 0.1)
    assert (LO.rmsnorm(x, torch.ones(96), 0.1).double() - wrong).abs().max() > 1e-2


def test_rope_oracle_invariants():
    gen = torch.Generator().manual_seed(1)
    D, T = 64, 50
    cos, sin = LO.rope_tables(4096, D, 1e6)
    x = torch.randn(2, 3, T, D, generator=gen)
    y = LO.apply_rope(x, cos[100 : 100 + T], sin[100 : 100 + T])
    # each (d, d + D/2) pair is rotated: its norm is preserved
    n_in = x[..., : D // 2] ** 2 + x[..., D // 2 :] ** 2
    n_out = y[..., : D // 2] ** 2 + y[..., D // 2 :] ** 2
    torch.testing.assert_close(n_out, n_in, rtol=1e-4, atol=1e-5)
    # position 0 is the identity
    torch.testing.assert_close(LO.apply_rope(x[:, :, :1], cos[:1], sin[:1]), x[:, :, :1])
    # explicit 2x2 rotation of pair j by angle p * base^(-2j/D)
    p, j = 137, 9
    ang = p * (1e6 ** (-2.0 * j / D))
    v = torch.randn(1, 1, 1, D, generator=gen)
    r = LO.apply_rope(v, cos[p : p + 1], sin[p : p + 1])
    a, b = v[0, 0, 0, j].item(), v[0, 0, 0, j + D // 2].item()
    assert r[0, 0, 0, j].item() == pytest.approx(a * math.cos(ang) - b * math.sin(ang), abs=1e-4)
    assert r[0, 0, 0, j + D // 2].item() == pytest.approx(b * math.cos(ang) + a * math.sin(ang), abs=1e-4)
    # q.k after rotation depends on the position difference only
    q, k = torch.randn(1, 1, 1, D, generator=gen), torch.randn(1, 1, 1, D, generator=gen)

    def dot(pq, pk):
        return (LO.apply_rope(q, cos[pq : pq + 1], sin[pq : pq + 1]) * LO.apply_rope(k, cos[pk : pk + 1], sin[pk : pk + 1])).sum().item()

    assert dot(10, 3) == pytest.approx(dot(1010, 1003), rel=1e-3, abs=1e-3)
    # and agrees with the rotary encoding used to build the attention benchmark inputs
    torch.testing.assert_close(y, O.apply_rope(x, torch.arange(100, 100 + T)), rtol=1e-5, atol=1e-5)


# ---- GPU ------------------------------------------------------------------------------------------------


@pytest.mark.gpu
@pytest.mark.parametrize("rows,dim", [(5, 64), (1024, 2560), (3, 8192), (17, 200), (7, 2048), (100, 4104), (20000, 2048)])
def test_rmsnorm_kernel(gpu, rows, dim):
    from keys_values_amd.longctx import ops

    gen = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, dim, generator=gen) * 3).to(torch.bfloat16)
    w = torch.rand(dim, generator=gen) + 0.5
    y = ops.rmsnorm(x.to(gpu), w.to(gpu), 1e-6).cpu()
    ref = LO.rmsnorm(x, w, 1e-6)
    # same arithmetic up to the order of the sum of squares: at most the last bf16 bit differs
    torch.testing.assert_close(y.float(), ref.float(), rtol=2 ** -7, atol=1e-6)
    assert (y != ref).float().mean().item() < 0.02


@pytest.mark.gpu
@pytest.mark.parametrize("rows,dim", [(5, 64), (1024, 2560), (3, 8192), (17, 200), (7, 2048), (100, 4104), (20000, 2048)])
def test_add_rmsnorm_kernel(gpu, rows, dim):
    # x = x + delta (rounded to bf16), then RMSNorm(x): the two separate steps of the oracle
    from keys_values_amd.longctx import ops

    gen = torch.Generator().manual_seed(rows * dim)
    x = (torch.randn(2, rows, dim, generator=gen) * 3).to(torch.bfloat16)
    delta = torch.randn(2, rows, dim, generator=gen).to(torch.bfloat16)
    w = torch.rand(dim, generator=gen) + 0.5
    xg = x.to(gpu)
    y = ops.add_rmsnorm_(xg, delta.to(gpu), w.to(gpu), 1e-6).cpu()
    x_ref = x + delta
    assert torch.equal(xg.cpu(), x_ref), "the residual stream must hold the rounded sum"
    ref = LO.rmsnorm(x_ref, w, 1e-6)
    torch.testing.assert_close(y.float(), ref.float(), rtol=2 ** -7, atol=1e-6)
    assert (y != ref).float().mean().item() < 0.02


@pytest.mark.gpu
@pytest.mark.parametrize("rows,dim", [(7, 16), (1024, 9728), (33, 200)])
def test_swiglu_kernel(gpu, rows, dim):
    # silu(gate) * up with the activation rounded to bf16 before the product, as F.silu(g) * u rounds
    import torch.nn.functional as F

    from keys_values_amd.longctx import ops

    gen = torch.Generator().manual_seed(dim)
    gu = (torch.randn(rows, 2 * dim, generator=gen) * 2).to(torch.bfloat16)
    gu[0, :4] = torch.tensor([0.0, -30.0, 30.0, -100.0]).to(torch.bfloat16)  # silu(0) = 0, tails: exp under / overflow
    out = ops.swiglu(gu.to(gpu)).cpu()
    ref = F.silu(gu[:, :dim]) * gu[:, dim:]
    torch.testing.assert_close(out.float(), ref.float(), rtol=2 ** -7, atol=1e-6)
    assert (out != ref).float().mean().item() < 0.01  # exp implementations differ in the last fp32 bits
    # closed form in float64 of the un-rounded function
    g64, u64 = gu[:, :dim].double(), gu[:, dim:].double()
    exact = g64 / (1 + torch.exp(-g64)) * u64
    torch.testing.assert_close(out.double(), exact, rtol=2 ** -6, atol=1e-6)
    assert torch.isfinite(out.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("B,num,Hq,Hkv,D,norm,input_pos", [(1, 64, 8, 2, 64, True, 0), (2, 100, 32, 8, 128, True, 4000), (1, 33, 4, 4, 128, False, 77)])
def test_qk_norm_rope_kernel(gpu, B, num, Hq, Hkv, D, norm, input_pos):
    from keys_values_amd.longctx import ops

    gen = torch.Generator().manual_seed(num)
    qkv = (torch.randn(B, num, (Hq + 2 * Hkv) * D, generator=gen) * 2).to(torch.bfloat16)
    qw = (torch.rand(D, generator=gen) + 0.5) if norm else None
    kw = (torch.rand(D, generator=gen) + 0.5) if norm else None
    cos, sin = LO.rope_tables(8192, D, 1e6)
    q_ref, k_ref, v_ref = LO.qk_norm_rope(qkv, Hq, Hkv, D, qw, kw, 1e-6, cos, sin, input_pos)
    g = qkv.to(gpu)
    cg, sg = ops.rope_tables(8192, D, 1e6, gpu)
    ops.qk_norm_rope_(g, Hq, Hkv, D, None if qw is None else qw.to(gpu), None if kw is None else kw.to(gpu), 1e-6, cg, sg, input_pos)
    out = g.cpu()
    q = out[..., : Hq * D].view(B, num, Hq, D).transpose(1, 2)
    k = out[..., Hq * D : (Hq + Hkv) * D].view(B, num, Hkv, D).transpose(1, 2)
    v = out[..., (Hq + Hkv) * D :].view(B, num, Hkv, D).transpose(1, 2)
    assert torch.equal(v, v_ref), "value heads must not be touched"
    for a, r in ((q, q_ref), (k, k_ref)):
        torch.testing.assert_close(a.float(), r.float(), rtol=2 ** -6, atol=2e-3)
        assert (a != r).float().mean().item() < 0.03  # device cos/sin and sum order: rare last-bit differences


@pytest.mark.gpu
@pytest.mark.parametrize("quantized", [False, True])
def test_prefill_model_vs_oracle(gpu, quantized):
    """Two layers, 8/2 heads of 64, cache of 256 slots, chunks of 64: the prefill chunk, the chunk under
    the initial rule and two H2O chunks. The caches are kept on the oracle's slots so that a near-tie in
    one layer's selection does not turn into a different trajectory (the selection itself is compared)."""
    from keys_values_amd.longctx.model import LongContextPrefillModel, PrefillConfig

    cfg = PrefillConfig(n_layer=2, n_embd=256, n_head=8, n_query_groups=2, head_size=64, intermediate_size=512, vocab_size=1000)
    L, chunk, B = 256, 64, 1
    model = LongContextPrefillModel(cfg, cache_length=L, chunk_size=chunk, max_batch_size=B, quantized=quantized, max_context=2048, seed=4, device=gpu)
    weights = [{k: getattr(layer, k).cpu() for k in ("qkv", "proj", "fc_1", "fc_2", "mlp_proj", "norm_1", "norm_2", "norm_q", "norm_k")}
               for layer in model.layers]
    ref = LO.PrefillOracle(cfg, model.wte.cpu(), weights, model.ln_f.cpu(), L, chunk, B, quantized, 2048)
    ids = torch.randint(0, cfg.vocab_size, (B, L + 3 * chunk), generator=torch.Generator().manual_seed(5))
    sizes = model.chunk_sizes(ids.shape[1])
    assert sizes == [L, chunk, chunk, chunk]
    model.reset()
    start = 0
    for ci, n in enumerate(sizes):
        sl = ids[:, start : start + n]
        forced = None
        if ci >= 2:
            # compare the device's choice with the oracle's, then continue on the oracle's slots
            forced = []
            for li, cache in enumerate(model.caches):
                want = ref.caches[li].next_index
                got = cache._next_index[:B].cpu().long()
                for h in range(cfg.n_query_groups):
                    a, r = set(got[0, h, :chunk].tolist()), set(want[0, h, :chunk].tolist())
                    assert len(a ^ r) <= 4, f"layer {li} head {h}: selections differ in {len(a ^ r)} slots"
                cache._next_index[:B, :, :chunk] = want[:, :, :chunk].to(torch.int32).to(gpu)
                forced.append(None)
        h_ref = ref.forward_chunk(sl, forced)
        h_gpu = model.forward_chunk(sl.to(gpu)).cpu()
        err = ((h_gpu.float() - h_ref.float()).norm() / h_ref.float().norm()).item()
        assert err < 3e-2, f"chunk {ci}: hidden states differ by {err}"
        for li, cache in enumerate(model.caches):
            assert torch.equal(cache.token_pos.cpu(), ref.caches[li].token_pos)
        start += n
