"""Pins the CPU oracle (oracle/kvx_oracle.py, oracle/kvx_oracle.c) without importing the reference:
brute force in float64, library routines on special cases, closed forms, the invariants and
cross-implementation checks the reference's own tests use, and hand-computed vectors."""
import math

import numpy as np
import pytest
import torch

from helpers import make_qkv, scattered_positions
from oracle import c_oracle as C
from oracle import kvx_oracle as O


@pytest.mark.parametrize("B,Hq,Hkv,q_len,T,D,input_pos", [(1, 4, 2, 5, 24, 8, 19), (2, 6, 2, 7, 20, 16, 30), (1, 3, 3, 4, 9, 4, 5)])
def test_sdpa_vs_bruteforce_f64(B, Hq, Hkv, q_len, T, D, input_pos):
    # formula of test/attention/test_attn_weights.py:51-101 as explicit float64 loops
    q, k, v, gen = make_qkv(11, B, Hq, Hkv, q_len, T, D, dtype=torch.float32)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    scale = 1.0 / math.sqrt(D)
    o_bf, w_bf, l_bf = O.weights_bruteforce_f64(q, k, v, scale, input_pos, tp)
    for fn in (O.sdpa_in_blocks, O.sdpa_noblock):
        o, w = fn(q, k, v, scale, input_pos, tp.to(torch.int64))
        np.testing.assert_allclose(o.numpy(), o_bf, rtol=2e-5, atol=2e-6)
        np.testing.assert_allclose(w.numpy(), w_bf, rtol=2e-5, atol=2e-7)
    np.testing.assert_allclose(O.lse2(q, k, scale, input_pos, tp).numpy(), l_bf, rtol=1e-5, atol=1e-5)
    oc, wc, lc = C.sdpa_weights(q.numpy(), k.numpy(), v.numpy(), tp.numpy(), input_pos, scale)
    np.testing.assert_allclose(oc, o_bf, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(wc, w_bf, rtol=2e-5, atol=2e-7)
    np.testing.assert_allclose(lc, l_bf, rtol=1e-5, atol=1e-5)


def test_mask_direction_is_pinned():
    # One query at position 5; slots hold positions 3, 5, 6. Visible iff position <= 5
    # (keys_values/attention/attention_utils.py:238-247). A flipped comparison or an off-by-one
    # changes which weights are zero.
    q = torch.ones(1, 1, 1, 2)
    k = torch.zeros(1, 1, 3, 2)
    v = torch.eye(3, 2).view(1, 1, 3, 2)
    tp = torch.tensor([[[3, 5, 6]]])
    _, w = O.sdpa_in_blocks(q, k, v, 1.0, 5, tp)
    assert torch.allclose(w, torch.tensor([[[0.5, 0.5, 0.0]]]))


def test_square_case_is_library_causal_sdpa():
    # T == q_len, positions = arange: the path reduces to causal SDPA, a library routine
    q, k, v, _ = make_qkv(3, 2, 4, 4, 33, 33, 16, dtype=torch.float32)
    o, w = O.sdpa_in_blocks(q, k, v, 0.25, 0, None)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.25)
    torch.testing.assert_close(o, ref, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(w.sum(-1), torch.full((2, 4), 33.0), rtol=1e-5, atol=1e-4)


def test_uniform_keys_closed_form():
    # identical keys -> uniform softmax over the visible slots: W[k] = sum_i 1 / #visible(i) over the
    # queries i that see k; O = mean of the visible values
    B, Hq, Hkv, q_len, T, D, input_pos = 1, 2, 1, 6, 16, 8, 10
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(B, Hq, q_len, D, generator=gen)
    k = torch.randn(1, 1, 1, D, generator=gen).expand(B, Hkv, T, D).contiguous()
    v = torch.randn(B, Hkv, T, D, generator=gen)
    o, w = O.sdpa_in_blocks(q, k, v, 0.3, input_pos, None)
    expect = torch.zeros(T)
    for i in range(q_len):
        nvis = input_pos + i + 1
        expect[:nvis] += 1.0 / nvis
    torch.testing.assert_close(w[0, 0], expect, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(o[0, 1, 2], v[0, 0, : input_pos + 3].mean(0), rtol=1e-5, atol=1e-6)


def test_single_query_is_a_softmax_row():
    q, k, v, _ = make_qkv(8, 2, 4, 2, 1, 50, 16, dtype=torch.float32)
    o, w = O.sdpa_in_blocks(q, k, v, 0.25, 49, None)
    s = torch.einsum("bhd,bhtd->bht", q[:, :, 0], k.repeat_interleave(2, dim=1)) * 0.25
    p = torch.softmax(s, -1)
    torch.testing.assert_close(w, p.view(2, 2, 2, 50).mean(2), rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(o[:, :, 0], torch.einsum("bht,bhtd->bhd", p, v.repeat_interleave(2, dim=1)), rtol=1e-5, atol=1e-6)


def test_invariants_nonneg_and_row_sums():
    # test/attention/test_flashinfer_wrapper.py:420-454
    q, k, v, gen = make_qkv(21, 2, 8, 2, 17, 96, 32, dtype=torch.float32)
    tp = scattered_positions(gen, 2, 2, 96, 200, 17)
    _, w = O.sdpa_in_blocks(q, k, v, 0.2, 200, tp.to(torch.int64))
    assert w.dtype == torch.float32 and w.shape == (2, 2, 96)
    assert (w >= 0).all()
    torch.testing.assert_close(w.sum(-1), torch.full((2, 2), 17.0), atol=3e-4, rtol=5e-5)


def test_gqa_is_mean_over_group():
    # test/attention/test_attention.py:78-166: GQA == repeat_interleave'd keys, weights averaged over the group
    q, k, v, _ = make_qkv(4, 1, 8, 2, 9, 40, 16, dtype=torch.float32)
    o, w = O.sdpa_in_blocks(q, k, v, 0.25, 31, None)
    o2, w2 = O.sdpa_in_blocks(q, k.repeat_interleave(4, dim=1), v.repeat_interleave(4, dim=1), 0.25, 31, None)
    torch.testing.assert_close(o, o2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(w, w2.view(1, 2, 4, 40).mean(2), rtol=1e-5, atol=1e-7)


def test_blocked_equals_unblocked():
    # test/attention/test_attention.py:706-797
    q, k, v, gen = make_qkv(6, 2, 4, 2, 40, 64, 16, dtype=torch.float32)
    tp = scattered_positions(gen, 2, 2, 64, 70, 40)
    o1, w1 = O.sdpa_in_blocks(q, k, v, 0.25, 70, tp.to(torch.int64), tmp_array_limit_gb=1e-5)  # forces many slices
    o2, w2 = O.sdpa_noblock(q, k, v, 0.25, 70, tp.to(torch.int64))
    assert O._tmp_len(2, 4, 40, 64, 1e-5) < 40
    torch.testing.assert_close(o1, o2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(w1, w2, rtol=1e-5, atol=1e-6)


def test_reorder_equals_position_mask():
    # test/attention/test_sdpa_wrapper.py:55-153: sorting the slots by position and applying a
    # right-aligned causal mask gives the same result as masking by token position
    B, Hq, Hkv, q_len, T, D, input_pos = 2, 4, 2, 12, 48, 16, 60
    q, k, v, gen = make_qkv(9, B, Hq, Hkv, q_len, T, D, dtype=torch.float32)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    o1, w1 = O.sdpa_in_blocks(q, k, v, 0.25, input_pos, tp.to(torch.int64))
    ks, vs, idx = O.reorder_key_value(k, v, tp)
    o2, w2s = O.sdpa_in_blocks(q, ks, vs, 0.25, T - q_len, None)
    w2 = torch.zeros_like(w2s).scatter_(-1, idx, w2s)
    torch.testing.assert_close(o1, o2, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(w1, w2, rtol=1e-5, atol=1e-6)


# ---- quantiser -------------------------------------------------------------------------------------


def test_quantiser_hand_vector():
    # scale = 4/255; zp = -rint(-1/scale) = -rint(-63.75) = 64; codes rint(x/scale) + 64
    x = torch.tensor([[-1.0, 0.0, 1.0, 3.0]])
    c, s, z = O.quantize_rows(x)
    assert c.tolist() == [[0, 64, 128, 255]]
    assert z.tolist() == [64]
    assert s.item() == np.float32(4.0) / np.float32(255.0)
    # half-to-even: 0.5/1 with scale 1 -> codes of [0, 0.5, 1.5, 2.5, 255] are [0, 0, 2, 2, 255]
    x = torch.tensor([[0.0, 0.5, 1.5, 2.5, 255.0]])
    c, s, z = O.quantize_rows(x)
    assert s.item() == 1.0 and z.item() == 0 and c.tolist() == [[0, 0, 2, 2, 255]]


def test_quantiser_constant_row_uses_eps():
    x = torch.full((1, 8), 1.0)
    c, s, z = O.quantize_rows(x)
    assert s.item() == np.float32(1.1920929e-07)
    assert z.item() == -8388608 and (c == 0).all()
    assert (O.dequantize_rows(c, s, z, torch.float32) == 1.0).all()


@pytest.mark.parametrize("kind", ["as_is", "shift", "scale", "shift_scale"])
def test_quantiser_known_answer_roundtrip(kind):
    # test/kvcache/test_quantization.py:647-766: integers in [0, 255] holding both extremes in every
    # row survive quantise -> dequantise (exactly unless scaled)
    gen = torch.Generator().manual_seed(31415927)
    shape = (3, 4, 32, 64)
    data = torch.randint(0, 256, shape, generator=gen)
    i0 = torch.randint(0, 64, shape[:-1], generator=gen)
    i1 = (i0 + 1 + torch.randint(0, 63, shape[:-1], generator=gen)) % 64
    data.scatter_(-1, i0.unsqueeze(-1), 0)
    data.scatter_(-1, i1.unsqueeze(-1), 255)
    x = data.to(torch.float32)
    if "shift" in kind:
        x = x + torch.randint(-1024, 1024, shape[:-1], generator=gen).unsqueeze(-1)
    if "scale" in kind:
        x = x * torch.randn(shape[:-1], generator=gen).exp().unsqueeze(-1)
    c, s, z = O.quantize_rows(x)
    back = O.dequantize_rows(c, s, z, torch.float32)
    if kind in ("as_is", "shift"):
        assert torch.equal(back, x)
        assert torch.equal(c.to(torch.int64), data)
    elif kind == "scale":
        torch.testing.assert_close(back, x)
    else:
        torch.testing.assert_close(back, x, rtol=1e-5, atol=0.025)


def test_quantiser_python_and_c_bit_equal():
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(4096, 128, generator=gen)
    mask = torch.rand(4096, 128, generator=gen) < 0.01
    x = torch.where(mask, torch.randn(4096, 128, generator=gen) * 8, x).to(torch.bfloat16)
    x[0] = 0.0
    x[1] = -3.5
    x[2, :64] = 1e-3
    c, s, z = O.quantize_rows(x)
    c2, s2, z2 = C.quantize_rows(x.float().numpy())
    assert np.array_equal(c.numpy(), c2) and np.array_equal(s.numpy(), s2) and np.array_equal(z.numpy(), z2)
    d = O.dequantize_rows(c, s, z, torch.float32)
    assert np.array_equal(d.numpy(), C.dequantize_rows(c2, s2, z2))
    # quantisation error is bounded by half a step (plus bf16 inputs are exact in fp32)
    assert ((x.float() - d).abs() <= 0.5001 * s.unsqueeze(-1) + 1e-7).all()


def test_quantization_error_bound_and_zero():
    # integers 0..255 with both extremes are represented exactly -> zero error; otherwise every
    # element is off by at most half a quantisation step
    x = torch.arange(256, dtype=torch.float32).view(2, 128)
    x[1] = x[0]
    x[1, 0], x[1, 127] = 0.0, 255.0
    assert (O.quantization_error(torch.stack((x[0] * 2, x[1]))[1:]) == 0).all()
    g = torch.Generator().manual_seed(1)
    y = torch.randn(64, 128, generator=g)
    _, s, _ = O.quantize_rows(y)
    err = O.quantization_error(y)
    assert (err <= 0.5001 * s * math.sqrt(128)).all() and (err > 0).all()


def test_quantiser_4bit_hand_vector_and_packing():
    # scale = 3/15 = 0.2; zp = -rint(-1/0.2) = 5; codes rint(x/0.2) + 5
    x = torch.tensor([[-1.0, -0.6, 0.0, 2.0]])
    c, s, z = O.quantize_rows(x, num_bits=4)
    assert c.tolist() == [[0, 2, 5, 15]] and z.tolist() == [5]
    assert s.item() == np.float32(3.0) / np.float32(15.0)
    # keys_values/kvcache/quantize/pytorch.py:384-393: first half of the row in the high nibbles
    assert O.compress4(c).tolist() == [[0 << 4 | 5, 2 << 4 | 15]]
    assert torch.equal(O.uncompress4(O.compress4(c)), c)
    codes = torch.arange(16, dtype=torch.uint8).view(1, 16)
    assert O.compress4(codes).tolist() == [[0x08, 0x19, 0x2A, 0x3B, 0x4C, 0x5D, 0x6E, 0x7F]]


@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("blocks_over_heads", [False, True])
@pytest.mark.parametrize("kind", ["as_is", "shift", "scale"])
def test_quantiser_store_known_answer(num_bits, blocks_over_heads, kind):
    # test/kvcache/test_quantization.py:647-766 for both widths and both block shapes: integers that
    # hold both extremes in every head row (hence in every block) round-trip exactly
    gen = torch.Generator().manual_seed(31415927)
    shape = (3, 4, 32, 64)
    high = 2**num_bits
    data = torch.randint(0, high, shape, generator=gen)
    i0 = torch.randint(0, 64, shape[:-1], generator=gen)
    i1 = (i0 + 1 + torch.randint(0, 63, shape[:-1], generator=gen)) % 64
    data.scatter_(-1, i0.unsqueeze(-1), 0)
    data.scatter_(-1, i1.unsqueeze(-1), high - 1)
    x = data.to(torch.float32)
    per_block = (3, 1, 32, 1) if blocks_over_heads else (3, 4, 32, 1)
    if kind == "shift":
        x = x + torch.randint(-1024, 1024, per_block, generator=gen)
    if kind == "scale":
        x = x * torch.randn(per_block, generator=gen).exp()
    buf, s, z = O.quantize_store(x, num_bits, blocks_over_heads)
    first, final = (3, 4 * 64) if blocks_over_heads else (12, 64)
    assert buf.shape == (first, 32, final * num_bits // 8) and buf.dtype == torch.uint8
    assert s.shape == (first, 32) and z.shape == (first, 32) and z.dtype == torch.int32
    back = O.dequantize_store(buf, s, z, shape, num_bits, blocks_over_heads, torch.float32)
    if kind == "scale":
        torch.testing.assert_close(back, x)
    else:
        assert torch.equal(back, x)
        codes = O.uncompress4(buf) if num_bits == 4 else buf
        want = data.transpose(1, 2).reshape(3, 32, 256) if blocks_over_heads else data.reshape(12, 32, 64)
        assert torch.equal(codes.to(torch.int64), want)


def test_quantiser_4bit_python_and_c_bit_equal():
    gen = torch.Generator().manual_seed(5)
    x = (torch.randn(2048, 128, generator=gen) * 2).to(torch.bfloat16)
    x[0] = 0.0
    x[1] = -3.5
    for E in (128, 1024):  # rows, and blocks over 8 heads
        xb = x.float().reshape(-1, E)
        c, s, z = O.quantize_rows(xb, num_bits=4)
        p = O.compress4(c)
        p2, s2, z2 = C.quantize_blocks4(xb.numpy())
        assert np.array_equal(p.numpy(), p2) and np.array_equal(s.numpy(), s2) and np.array_equal(z.numpy(), z2)
        d = O.dequantize_rows(O.uncompress4(p), s, z, torch.float32)
        assert np.array_equal(d.numpy(), C.dequantize_blocks4(p2, s2, z2))
        assert ((xb - d).abs() <= 0.5001 * s.unsqueeze(-1) + 1e-7).all()


# ---- H2O bookkeeping -------------------------------------------------------------------------------


def test_select_smallest_bruteforce_and_c():
    gen = torch.Generator().manual_seed(7)
    scores = torch.rand(2, 3, 40, generator=gen)
    scores[0, 0, 5] = scores[0, 0, 17]  # an exact tie: lower slot first
    w = torch.rand(2, 3, 36, generator=gen)
    s_py = scores.clone()
    nxt = O.h2o_update_select(s_py, w, 36, 38, 9)
    s_c = scores.numpy().copy()
    nxt_c = C.h2o_update_select(s_c, w.numpy(), 36, 38, 9)
    assert np.array_equal(nxt.numpy(), nxt_c)
    np.testing.assert_array_equal(s_py.numpy(), s_c)
    # brute force: python sort of (value, slot)
    for b in range(2):
        for h in range(3):
            row = [(s_py[b, h, t].item(), t) for t in range(38)]
            assert [t for _, t in sorted(row)[:9]] == nxt[b, h].tolist()


def test_h2o_cache_oracle_bookkeeping():
    # test/kvcache/test_h2o.py:109-137,227-343 and test/kvcache/test_generic.py:53-116 restated:
    # cumulative scores are the running sum of the per-step weights with a reset on overwrite,
    # every slot holds the K/V of the token token_pos names, positions are unique, and the slots
    # written are the first `num` of the previous selection.
    B, Hq, Hkv, L, D = 2, 4, 2, 32, 8
    gen = torch.Generator().manual_seed(13)
    cache = O.H2OCacheOracle(B, Hq, Hkv, L, D)
    total = 32 + 5 * 6
    qs = torch.randn(B, Hq, total, D, generator=gen)
    ks = torch.randn(B, Hkv, total, D, generator=gen)
    vs = torch.randn(B, Hkv, total, D, generator=gen)
    cache.prefill(qs[:, :, :32], ks[:, :, :32], vs[:, :, :32])
    expect_scores = torch.zeros(B, Hkv, L)
    pos = 32
    prev_next = None
    for step in range(5):
        sl = slice(pos, pos + 6)
        o, w, index = cache.forward(qs[:, :, sl], ks[:, :, sl], vs[:, :, sl])
        if step == 0:
            assert index[0, 0].tolist() == list(range(1, 7))  # int(0.05 * 32) = 1: the initial rule
        else:
            assert torch.equal(index, prev_next[:, :, :6])
        expect_scores.scatter_(-1, index, 0.0)
        expect_scores += w
        torch.testing.assert_close(cache.scores, expect_scores, rtol=5e-3, atol=5e-3)
        torch.testing.assert_close(w.sum(-1), torch.full((B, Hkv), 6.0), rtol=1e-4, atol=1e-4)
        prev_next = cache.next_index
        assert torch.equal(prev_next, torch.argsort(cache.scores, dim=-1, stable=True))
        pos += 6
        for b in range(B):
            for h in range(Hkv):
                tp = cache.token_pos[b, h].long()
                assert len(set(tp.tolist())) == L
                assert torch.equal(cache.k[b, h], ks[b, h, tp])
                assert torch.equal(cache.v[b, h], vs[b, h, tp])
