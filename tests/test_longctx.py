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


def _schedule_by_walk(mpl, lengths, seq, chunk):
    """Checker: the reference's cursor walk (keys_values/long_context.py:72-113, deterministic branch)."""
    cuts = sorted(set(c for c in lengths if c <= seq))
    if not cuts:
        return [seq] if mpl >= seq else [mpl, seq - mpl]
    out, done = [mpl], mpl
    while done < seq:
        size = min(chunk, seq - done)
        if cuts and done + size >= cuts[0] - 4:
            size = cuts.pop(0) - done
        if size > 0:
            out.append(size)
        done += size
    return out


def test_chunk_sizes_equal_the_cursor_walk_on_random_cases():
    import random

    rnd = random.Random(7)
    for _ in range(3000):
        chunk = rnd.choice([1, 2, 3, 4, 5, 7, 16, 64, 100, 1024])
        mpl = rnd.randint(1, 300)
        lengths = [mpl + rnd.randint(0, 400) for _ in range(rnd.randint(1, 4))]
        seq = rnd.randint(1, 1500)
        assert create_chunk_sizes(mpl, lengths, seq, chunk) == _schedule_by_walk(mpl, lengths, seq, chunk), (mpl, lengths, seq, chunk)
    with pytest.raises(ValueError):
        create_chunk_sizes(100, [50], 200, 16)


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


def _bf16_round(x: float) -> float:
    """Round-to-nearest-even of a Python float to bfloat16, by hand on the fp32 bit pattern."""
    import struct

    bits = struct.unpack("<I", struct.pack("<f", x))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def test_qk_norm_rope_oracle_against_per_head_loops():
    """keys_values/model.py:686-775: the projection's output holds, per token, n_head query heads, then
    n_query_groups key heads, then as many value heads; queries are normalised with norm_q, keys with
    norm_k (per head, over head_size), the result is rounded to the activations' type, then rotated by
    the token's own position input_pos + t, and rounded again; values pass through."""
    B, num, Hq, Hkv, D, input_pos, eps = 2, 5, 4, 2, 16, 37, 1e-6
    gen = torch.Generator().manual_seed(8)
    qkv = (torch.randn(B, num, (Hq + 2 * Hkv) * D, generator=gen) * 2).to(torch.bfloat16)
    qw, kw = torch.rand(D, generator=gen) + 0.5, torch.rand(D, generator=gen) + 0.5
    cos, sin = LO.rope_tables(256, D, 1e4)
    q, k, v = LO.qk_norm_rope(qkv, Hq, Hkv, D, qw, kw, eps, cos, sin, input_pos)
    assert q.shape == (B, Hq, num, D) and k.shape == (B, Hkv, num, D) and v.shape == (B, Hkv, num, D)
    # (1) composition from the pinned pieces, one (token, head) row at a time
    for b in range(B):
        for t in range(num):
            p = input_pos + t
            for h in range(Hq + 2 * Hkv):
                row = qkv[b, t, h * D : (h + 1) * D]
                if h < Hq:
                    want = LO.apply_rope(LO.rmsnorm(row.view(1, D), qw, eps), cos[p : p + 1], sin[p : p + 1])[0]
                    assert torch.equal(q[b, h, t], want), (b, t, h)
                elif h < Hq + Hkv:
                    want = LO.apply_rope(LO.rmsnorm(row.view(1, D), kw, eps), cos[p : p + 1], sin[p : p + 1])[0]
                    assert torch.equal(k[b, h - Hq, t], want), (b, t, h)
                else:
                    assert torch.equal(v[b, h - Hq - Hkv, t], row), (b, t, h)
    # (2) scalar arithmetic in Python floats with both roundings written out, for every element of a few rows
    worst = 0.0
    differs_without_middle_round = False
    for (b, t, h) in ((0, 0, 0), (1, 3, 2), (0, 4, Hq), (1, 1, Hq + 1)):
        row = [float(x) for x in qkv[b, t, h * D : (h + 1) * D]]
        wt = qw if h < Hq else kw
        rms = math.sqrt(sum(x * x for x in row)) / math.sqrt(D)
        exact = [x / (rms + eps) * float(wt[d]) for d, x in enumerate(row)]
        normed = [_bf16_round(x) for x in exact]
        p = input_pos + t
        got = (q[b, h, t] if h < Hq else k[b, h - Hq, t]).tolist()
        for src, check in ((normed, True), (exact, False)):
            for d in range(D):
                j = d % (D // 2)
                ang = p * (1e4 ** (-2.0 * j / D))
                other = -src[d + D // 2] if d < D // 2 else src[d - D // 2]
                val = _bf16_round(src[d] * math.cos(ang) + other * math.sin(ang))
                if check:
                    worst = max(worst, abs(val - got[d]) / max(abs(val), 1e-3))
                elif val != got[d]:
                    differs_without_middle_round = True
    assert worst <= 2 ** -7, worst  # at most the last bf16 bit (fp32 cos/sin against float64 here)
    assert differs_without_middle_round, "the rounding between normalisation and rotation must be visible in the data"


def _tiny_prefill_setup(quantized, zero_out=False, seed=3):
    from types import SimpleNamespace

    cfg = SimpleNamespace(n_layer=1, n_embd=16, n_head=2, n_query_groups=1, head_size=8, intermediate_size=24, vocab_size=50,
                          rope_base=1e4, norm_eps=1e-5)
    gen = torch.Generator().manual_seed(seed)

    def w(o, i, std=0.3):
        return (torch.randn(o, i, generator=gen) * std).to(torch.bfloat16)

    d = cfg.head_size
    layer = dict(qkv=w((cfg.n_head + 2 * cfg.n_query_groups) * d, cfg.n_embd), proj=w(cfg.n_embd, cfg.n_head * d),
                 fc_1=w(cfg.intermediate_size, cfg.n_embd), fc_2=w(cfg.intermediate_size, cfg.n_embd),
                 mlp_proj=w(cfg.n_embd, cfg.intermediate_size), norm_1=torch.rand(cfg.n_embd, generator=gen) + 0.5,
                 norm_2=torch.rand(cfg.n_embd, generator=gen) + 0.5, norm_q=torch.rand(d, generator=gen) + 0.5,
                 norm_k=torch.rand(d, generator=gen) + 0.5)
    if zero_out:
        layer["proj"].zero_()
        layer["mlp_proj"].zero_()
    wte = w(cfg.vocab_size, cfg.n_embd, 1.0)
    ln_f = torch.rand(cfg.n_embd, generator=gen) + 0.5
    L, chunk = 8, 2
    ora = LO.PrefillOracle(cfg, wte, [layer], ln_f, L, chunk, 1, quantized, 64)
    ids = torch.randint(0, cfg.vocab_size, (1, L + 3 * chunk), generator=gen)
    return cfg, layer, wte, ln_f, L, chunk, ora, ids


def test_prefill_oracle_with_zero_output_projections_is_the_final_norm_of_the_embeddings():
    # both residual branches add exactly zero: the stack reduces to ln_f(wte[ids])
    cfg, layer, wte, ln_f, L, chunk, ora, ids = _tiny_prefill_setup(False, zero_out=True)
    start = 0
    for n in (L, chunk, chunk, chunk):
        sl = ids[:, start : start + n]
        assert torch.equal(ora.forward_chunk(sl), LO.rmsnorm(wte[sl], ln_f, cfg.norm_eps))
        start += n
    assert ora.input_pos == L + 3 * chunk and ora.caches[0].input_pos == ora.input_pos


@pytest.mark.parametrize("quantized", [False, True])
def test_prefill_oracle_one_layer_token_by_token(quantized):
    """One block on tiny widths recomputed token by token: explicit matrix-vector products in fp32
    rounded to bf16, the pinned row functions, and a cache oracle of its own fed chunk by chunk
    (Block.forward, keys_values/model.py:560-584, non-parallel residual: x += attn(norm_1 x);
    x += mlp(norm_2 x); CausalSelfAttention.forward, :686-811)."""
    cfg, layer, wte, ln_f, L, chunk, ora, ids = _tiny_prefill_setup(quantized)
    Hq, Hkv, D = cfg.n_head, cfg.n_query_groups, cfg.head_size
    cos, sin = LO.rope_tables(64, D, cfg.rope_base)
    cache = O.H2OCacheOracle(1, Hq, Hkv, L, D, dtype=torch.bfloat16, max_chunk_size=chunk)

    def matvec(W, x):  # bf16 weights and activations, fp32 accumulation, one rounding
        return torch.tensor([sum(float(a) * float(b) for a, b in zip(rowW, x)) for rowW in W.float()]).to(torch.bfloat16)

    def stored(x):
        return O.dequantize_rows(*O.quantize_rows(x)) if quantized else x

    start = 0
    for ci, n in enumerate((L, chunk, chunk, chunk)):
        sl = ids[:, start : start + n]
        got = ora.forward_chunk(sl)
        xs = [wte[int(i)] for i in sl[0]]
        q = torch.empty(1, Hq, n, D, dtype=torch.bfloat16)
        k = torch.empty(1, Hkv, n, D, dtype=torch.bfloat16)
        v = torch.empty(1, Hkv, n, D, dtype=torch.bfloat16)
        for t, x in enumerate(xs):
            qkv = matvec(layer["qkv"], LO.rmsnorm(x.view(1, -1), layer["norm_1"], cfg.norm_eps)[0])
            p = start + t
            for h in range(Hq):
                q[0, h, t] = LO.apply_rope(LO.rmsnorm(qkv[h * D : (h + 1) * D].view(1, D), layer["norm_q"], cfg.norm_eps), cos[p : p + 1], sin[p : p + 1])[0]
            for h in range(Hkv):
                o = (Hq + h) * D
                k[0, h, t] = LO.apply_rope(LO.rmsnorm(qkv[o : o + D].view(1, D), layer["norm_k"], cfg.norm_eps), cos[p : p + 1], sin[p : p + 1])[0]
                v[0, h, t] = qkv[o + Hkv * D : o + Hkv * D + D]
        if ci == 0:
            att = cache.prefill(q, k, v, stored(k), stored(v))
        else:
            att, _, _ = cache.forward(q, stored(k), stored(v))
        for t, x in enumerate(xs):
            y = torch.cat([att[0, h, t] for h in range(Hq)])  # heads side by side, keys_values/attention/base.py:378-380
            x = x + matvec(layer["proj"], y)
            xn = LO.rmsnorm(x.view(1, -1), layer["norm_2"], cfg.norm_eps)[0]
            g, u = matvec(layer["fc_1"], xn), matvec(layer["fc_2"], xn)
            act = (g.float() / (1.0 + torch.exp(-g.float()))).to(torch.bfloat16)  # silu, rounded as an op of its own
            x = x + matvec(layer["mlp_proj"], act * u)
            want = LO.rmsnorm(x.view(1, -1), ln_f, cfg.norm_eps)[0]
            torch.testing.assert_close(got[0, t].float(), want.float(), rtol=2 ** -6, atol=2 ** -7)
        assert torch.equal(cache.token_pos, ora.caches[0].token_pos) and torch.equal(cache.scores, ora.caches[0].scores)
        start += n


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
@pytest.mark.parametrize("B,num,Hq,Hkv,D,norm,input_pos", [(1, 64, 8, 2, 64, True, 0), (2, 100, 32, 8, 128, True, 4000), (1, 33, 4, 4, 128, False, 77), (2, 19, 4, 2, 256, True, 300)])
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
                cache.wait_for_selection()  # the choice runs on a second stream
                got = cache._next_index[:B].cpu().long()
                for h in range(cfg.n_query_groups):
                    a, r = set(got[0, h, :chunk].tolist()), set(want[0, h, :chunk].tolist())
                    assert len(a ^ r) <= 4, f"layer {li} head {h}: selections differ in {len(a ^ r)} slots"
                cache.set_next_positions(want[:, :, :chunk])
                forced.append(None)
        h_ref = ref.forward_chunk(sl, forced)
        h_gpu = model.forward_chunk(sl.to(gpu)).cpu()
        err = ((h_gpu.float() - h_ref.float()).norm() / h_ref.float().norm()).item()
        assert err < 3e-2, f"chunk {ci}: hidden states differ by {err}"
        for li, cache in enumerate(model.caches):
            assert torch.equal(cache.token_pos.cpu(), ref.caches[li].token_pos)
        start += n


@pytest.mark.gpu
def test_gemm_table_is_opt_in_and_restores_state(gpu, tmp_path):
    """Building the model does not touch TunableOp; a table PyTorch refuses (other library versions) leaves its
    switches as they were found."""
    import torch.cuda.tunable as tunable

    from keys_values_amd.longctx.model import LongContextPrefillModel, PrefillConfig, use_gemm_table

    def state():
        return tunable.is_enabled(), tunable.tuning_is_enabled(), tunable.record_untuned_is_enabled()

    before = state()
    cfg = PrefillConfig(n_layer=1, n_embd=128, n_head=4, n_query_groups=2, head_size=64, intermediate_size=256, vocab_size=100)
    model = LongContextPrefillModel(cfg, cache_length=128, chunk_size=64, max_batch_size=1, quantized=False, max_context=512, seed=4, device=gpu)
    assert model.gemm_table is False and state() == before
    bad = tmp_path / "mismatch.csv"
    bad.write_text("Validator,PT_VERSION,0.0.1\nValidator,HIP_VERSION,1\nGemmTunableOp_BFloat16_TN,tn_8_8_8_ld_8_8_8,Gemm_Rocblas_1,0.01\n")
    assert use_gemm_table(str(bad)) is False
    assert state() == before
    assert use_gemm_table(str(tmp_path / "absent.csv")) is False
    assert state() == before
