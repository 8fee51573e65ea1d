"""GPU parity of the attention kernels against the CPU oracle, through the C ABI (ctypes)."""
import ctypes
import math

import pytest
import torch

from helpers import make_qkv, rel_err, scattered_positions
from keys_values_amd import _lib
from keys_values_amd.attention import ops
from keys_values_amd.attention.sdpa import HipSDPA
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu

# tolerances of the path: outputs 2e-2 relative (bf16), score-sums 1e-3 relative (fp32 accumulation)
O_RTOL = 2e-2
W_RTOL = 1e-3


def check_o(o_gpu, o_ref):
    o_gpu = o_gpu.float().cpu()
    o_ref = o_ref.float()
    assert rel_err(o_gpu, o_ref) < O_RTOL
    torch.testing.assert_close(o_gpu, o_ref, rtol=O_RTOL, atol=2e-2)


def check_w(w_gpu, w_ref, q_len):
    w_gpu = w_gpu.cpu()
    assert w_gpu.dtype == torch.float32
    assert (w_gpu >= 0).all()
    torch.testing.assert_close(w_gpu, w_ref, rtol=W_RTOL, atol=1e-6)
    torch.testing.assert_close(w_gpu.sum(-1), torch.full(w_gpu.shape[:2], float(q_len)), rtol=5e-5, atol=3e-4)


CASES = [
    # B, Hq, Hkv, q_len, T, D, input_pos, scattered, splits
    (1, 8, 2, 128, 1024, 64, 896, False, 0),     # configuration 1 shapes
    (1, 8, 2, 128, 1024, 64, 896, True, 2),
    (2, 4, 4, 16, 200, 128, 300, True, 1),       # G = 1, ragged T
    (1, 8, 2, 100, 333, 128, 233, False, 3),     # ragged rows and keys, 3 splits
    (2, 8, 1, 37, 700, 128, 1000, True, 0),      # G = 8
    (1, 32, 8, 64, 192, 128, 128, False, 1),     # the reference's fused-prefill test shape
    (1, 4, 2, 2, 64, 64, 62, False, 1),
    (1, 4, 2, 300, 300, 128, 0, False, 2),       # square causal prefill (input_pos = 0)
]


@pytest.mark.parametrize("B,Hq,Hkv,q_len,T,D,input_pos,scattered,splits", CASES)
def test_prefill_with_weights(gpu, B, Hq, Hkv, q_len, T, D, input_pos, scattered, splits):
    q, k, v, gen = make_qkv(100 + T + q_len, B, Hq, Hkv, q_len, T, D)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len) if scattered else None
    if tp is None and input_pos != T - q_len:
        tp = (torch.arange(T, dtype=torch.int32) + (input_pos - (T - q_len))).view(1, 1, T).expand(B, Hkv, T).contiguous()
    scale = 1.0 / math.sqrt(D)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, None if tp is None else tp.to(torch.int64))
    l_ref = O.lse2(q, k, scale, input_pos, tp)
    out, w, lse = ops.prefill_core(
        q.to(gpu), k.to(gpu), v.to(gpu), scale, input_pos, None if tp is None else tp.to(gpu),
        return_weights=True, return_lse=True, output_transposed=False, num_splits=splits,
    )
    torch.cuda.synchronize()
    check_o(out, o_ref)
    torch.testing.assert_close(lse.cpu(), l_ref, rtol=1e-4, atol=1e-3)
    check_w(w, w_ref, q_len)


def test_prefill_strided_cache_views_and_layouts(gpu):
    # K/V as views k[:B, :, :T] of a larger (Bmax, Hkv, L, D) allocation
    # (keys_values/kvcache/buffers.py:538-541) and the extension's [B, len, H, D] layout
    B, Hq, Hkv, q_len, T, D, L = 2, 8, 2, 48, 160, 128, 256
    q, k, v, gen = make_qkv(5, B, Hq, Hkv, q_len, T, D)
    tp = scattered_positions(gen, B, Hkv, T, 400, q_len)
    scale = 0.09
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, 400, tp.to(torch.int64))
    kbuf = torch.zeros(3, Hkv, L, D, dtype=torch.bfloat16, device=gpu)
    vbuf = torch.zeros(3, Hkv, L, D, dtype=torch.bfloat16, device=gpu)
    tpbuf = torch.zeros(3, Hkv, L, dtype=torch.int32, device=gpu)
    kbuf[:B, :, :T] = k.to(gpu)
    vbuf[:B, :, :T] = v.to(gpu)
    tpbuf[:B, :, :T] = tp.to(gpu)
    out, w, _ = ops.prefill_core(q.to(gpu), kbuf[:B, :, :T], vbuf[:B, :, :T], scale, 400, tpbuf[:B, :, :T], return_weights=True)
    assert out.shape == (B, q_len, Hq, D)
    check_o(out.permute(0, 2, 1, 3), o_ref)
    check_w(w, w_ref, q_len)
    # reference extension layout, right-aligned causal
    o2_ref, w2_ref = O.sdpa_in_blocks(q, k, v, scale, T - q_len, None)
    out2, w2, lse2 = ops.sdpa_prefill(
        q.to(gpu).transpose(1, 2).contiguous(), k.to(gpu).transpose(1, 2).contiguous(), v.to(gpu).transpose(1, 2).contiguous(),
        scale, return_weights=True, return_lse=True,
    )
    check_o(out2.permute(0, 2, 1, 3), o2_ref)
    check_w(w2, w2_ref, q_len)
    torch.testing.assert_close(lse2.cpu(), O.lse2(q, k, scale, T - q_len, None), rtol=1e-4, atol=1e-3)


def test_score_sum_from_given_lse(gpu):
    # the score-sum kernel alone, fed the oracle's LSE (as the reference tests its Triton kernel,
    # test/attention/test_flashinfer_wrapper.py:1207-1307)
    B, Hq, Hkv, q_len, T, D = 1, 8, 2, 70, 530, 128
    q, k, v, gen = make_qkv(77, B, Hq, Hkv, q_len, T, D)
    tp = scattered_positions(gen, B, Hkv, T, 600, q_len)
    scale = 1.0 / math.sqrt(D)
    _, w_ref = O.sdpa_in_blocks(q, k, v, scale, 600, tp.to(torch.int64))
    lse = O.lse2(q, k, scale, 600, tp)
    w = ops.score_sum_core(q.to(gpu), k.to(gpu), lse.to(gpu), scale, 600, tp.to(gpu))
    check_w(w, w_ref, q_len)


@pytest.mark.parametrize("store", ["bf16", "u8"])
def test_score_sum_with_eight_wavefront_workgroups(gpu, store):
    # enough keys for the launch to take workgroups of 512 keys (8 KV heads x 32 workgroups), the last one
    # ragged, causal inside the chunk, scattered slots
    B, Hq, Hkv, q_len, T, D = 1, 16, 8, 40, 16000, 64
    q, k, v, gen = make_qkv(78, B, Hq, Hkv, q_len, T, D)
    input_pos = T + 11
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    scale = 1.0 / math.sqrt(D)
    quant, kg = None, k.to(gpu)
    if store == "u8":
        kc, ks, kz = O.quantize_rows(k)
        k = O.dequantize_rows(kc, ks, kz)
        kg = kc.to(gpu)
        quant = ops.QuantState(ks.to(gpu), kz.to(gpu), ks.to(gpu), kz.to(gpu))
    _, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, tp.to(torch.int64))
    lse = O.lse2(q, k, scale, input_pos, tp)
    w = ops.score_sum_core(q.to(gpu), kg, lse.to(gpu), scale, input_pos, tp.to(gpu), quant=quant)
    check_w(w, w_ref, q_len)
    torch.testing.assert_close(w.sum(-1).cpu(), torch.full((B, Hkv), float(q_len)), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("B,Hq,Hkv,q_len,T,D", [(1, 8, 2, 700, 900, 128), (2, 4, 1, 1100, 1100, 64), (1, 16, 2, 300, 2048, 128)])
def test_score_sum_over_split_query_rows(kvx, gpu, B, Hq, Hkv, q_len, T, D):
    # a short cache: with a workspace the query rows are split over several workgroups and the partial sums
    # added by a second launch; without one the kernel walks all rows. Both against the oracle, and each other.
    q, k, v, gen = make_qkv(79 + T, B, Hq, Hkv, q_len, T, D)
    input_pos = T - q_len + 3
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    scale = 1.0 / math.sqrt(D)
    _, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, tp.to(torch.int64))
    lse = O.lse2(q, k, scale, input_pos, tp).to(gpu)
    qg, kg, tpg = q.to(gpu), k.to(gpu), tp.to(gpu)
    w_split = ops.score_sum_core(qg, kg, lse, scale, input_pos, tpg)
    check_w(w_split, w_ref, q_len)
    a = _lib.SdpaArgs()
    ops._fill_common(a, qg, kg, None, scale, input_pos, tpg, None, 0)
    assert kvx.kvx_sdpa_prefill_workspace_bytes(ctypes.byref(a)) > 0  # the shape does split
    w_whole = torch.empty_like(w_split)
    a.lse, a.w = lse.data_ptr(), w_whole.data_ptr()
    _lib.check(kvx.kvx_score_sum(ctypes.byref(a), _lib.stream_ptr(gpu)))  # no workspace: no split
    torch.cuda.synchronize()
    check_w(w_whole, w_ref, q_len)
    torch.testing.assert_close(w_split, w_whole, rtol=1e-5, atol=1e-7)
    assert torch.equal(w_split, ops.score_sum_core(qg, kg, lse, scale, input_pos, tpg))  # the same bits every time


def test_causal_weights_decay(gpu):
    # test/attention/test_flashinfer_wrapper.py:1074-1124: early keys collect far more weight
    q, k, v, _ = make_qkv(3, 1, 8, 2, 64, 64, 64)
    _, w, _ = ops.prefill_core(q.to(gpu), k.to(gpu), v.to(gpu), 0.125, 0, None, return_weights=True)
    w = w.cpu()
    assert (w[:, :, 0] > 2 * w[:, :, -1]).all()


def test_hip_sdpa_dropin(gpu):
    # FlashInferSDPA surface incl. head-size padding (keys_values/attention/flashinfer_wrapper.py:276-308)
    B, Hq, Hkv, q_len, T, D = 1, 4, 2, 20, 90, 48
    q, k, v, gen = make_qkv(42, B, Hq, Hkv, q_len, T, D)
    tp = scattered_positions(gen, B, Hkv, T, 111, q_len)
    sdpa = HipSDPA()
    assert sdpa.available
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, 1 / math.sqrt(D), 111, tp.to(torch.int64))
    out, w = sdpa.scaled_dot_product_attention(q.to(gpu), k.to(gpu), v.to(gpu), None, 111, tp.to(gpu), return_attn_weights=True)
    assert out.shape == (B, Hq, q_len, D) and w.shape == (B, Hkv, T)
    check_o(out, o_ref)
    check_w(w, w_ref, q_len)
    out_t, w_none = sdpa.scaled_dot_product_attention(q.to(gpu), k.to(gpu), v.to(gpu), None, 111, tp.to(gpu), output_transposed=True)
    assert w_none is None and out_t.shape == (B, q_len, Hq, D)
    check_o(out_t.transpose(1, 2), o_ref)
    # q_len == 1 routes to the decode kernel and ignores positions
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], k, v, 1 / math.sqrt(D), 10**6, None)
    out1, w1 = sdpa.scaled_dot_product_attention(q[:, :, :1].to(gpu), k.to(gpu), v.to(gpu), None, 500, tp.to(gpu), return_attn_weights=True)
    check_o(out1, o1_ref)
    check_w(w1, w1_ref, 1)


DECODE_CASES = [
    # B, Hq, Hkv, T, D, splits
    (2, 8, 2, 1000, 128, 0),
    (1, 32, 8, 4096 + 77, 128, 0),
    (3, 4, 4, 130, 64, 1),
    (1, 8, 1, 5000, 128, 3),
    (2, 4, 2, 17, 64, 0),
    (1, 8, 2, 9000, 64, 2),
    (2, 6, 2, 700, 128, 0),        # group sizes that are not powers of two: 3, 7 (Qwen2-7B: 28 / 4), 5, 6
    (1, 28, 4, 3000, 128, 2),
    (1, 5, 1, 513, 64, 1),
    (2, 12, 2, 260, 128, 0),
    (1, 32, 2, 3000, 128, 0),      # 16 and 12 heads per KV head: both products on the matrix cores, 16 head columns
    (2, 24, 2, 700, 64, 0),
    (1, 16, 1, 1100, 64, 2),
]


@pytest.mark.parametrize("B,Hq,Hkv,T,D,splits", DECODE_CASES + [(2, 8, 2, 20000, 128, 0), (1, 8, 1, 9000, 64, 0), (1, 4, 2, 5000, 256, 0), (1, 16, 2, 4100, 128, 0)])
def test_decode_with_weights(gpu, decode_route, B, Hq, Hkv, T, D, splits):
    q, k, v, _ = make_qkv(900 + T, B, Hq, Hkv, 1, T, D)
    scale = 1.0 / math.sqrt(D)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, T - 1, None)
    l_ref = O.lse2(q, k, scale, T - 1, None)
    out, w, lse = ops.decode_core(q.to(gpu), k.to(gpu), v.to(gpu), scale, return_weights=True, return_lse=True, num_splits=splits)
    torch.cuda.synchronize()
    check_o(out.unsqueeze(2), o_ref)
    torch.testing.assert_close(lse.cpu(), l_ref, rtol=1e-4, atol=1e-3)
    check_w(w, w_ref, 1)
    # reference extension layout
    out2, w2 = ops.sdpa_decode(q[:, :, 0].to(gpu), k.to(gpu).transpose(1, 2).contiguous(), v.to(gpu).transpose(1, 2).contiguous(), scale, return_weights=True)
    check_o(out2.unsqueeze(2), o_ref)
    check_w(w2, w_ref, 1)
    out3, w3 = ops.sdpa_decode(q[:, :, 0].to(gpu), k.to(gpu).transpose(1, 2).contiguous(), v.to(gpu).transpose(1, 2).contiguous(), scale)
    assert w3 is None
    check_o(out3.unsqueeze(2), o_ref)


def test_decode_reports_the_splits_that_took_the_scratch_route(kvx, gpu):
    """The optional counter of a decode call: 0 when every split turned its own logits into weights, every split
    when that form is switched off or no split waits, and nothing written without score-sums."""
    B, Hq, Hkv, T, D = 2, 8, 2, 20000, 128
    q, k, v, _ = make_qkv(77, B, Hq, Hkv, 1, T, D)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    scale = 1.0 / math.sqrt(D)
    counts, ws = {}, {}
    try:
        for name, setting in (("resident", (-1, -1, -1)), ("scratch", (0, -1, -1)), ("no-wait", (-1, 0, -1))):
            kvx.kvx_decode_tuning(*setting)
            n = torch.full((1,), -5, dtype=torch.int32, device=gpu)
            _, ws[name], _ = ops.decode_core(qg, kg, vg, scale, return_weights=True, scratch_splits=n)
            counts[name] = int(n.item())
    finally:
        kvx.kvx_decode_tuning(-1, -1, -1)
    assert counts["resident"] == 0
    assert counts["scratch"] == counts["no-wait"] and counts["scratch"] >= B * Hkv and counts["scratch"] % (B * Hkv) == 0
    assert torch.equal(ws["resident"], ws["scratch"]) and torch.equal(ws["resident"], ws["no-wait"])
    n = torch.full((1,), -5, dtype=torch.int32, device=gpu)
    ops.decode_core(qg, kg, vg, scale, return_weights=False, scratch_splits=n)
    assert int(n.item()) == 0  # no logits, nothing through the scratch


def test_full_size_prefill_properties(gpu):
    """Configuration 2 at its real shape (B1, 32/8 heads, D128, 32768 slots, 1024 queries, RoPE):
    one KV head against the oracle, row sums, and layout independence (scattered slots give the
    same O and, after un-permuting, the same W as the contiguous layout)."""
    B, Hq, Hkv, q_len, T, D, input_pos = 1, 32, 8, 1024, 32768, 128, 31744
    gen = torch.Generator().manual_seed(1)
    q = torch.randn(B, Hq, q_len, D, generator=gen)
    k = torch.randn(B, Hkv, T, D, generator=gen)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16)
    q = O.apply_rope(q, torch.arange(input_pos, input_pos + q_len)).to(torch.bfloat16)
    k = O.apply_rope(k, torch.arange(T)).to(torch.bfloat16)
    scale = D ** -0.5
    out, w, lse = ops.prefill_core(q.to(gpu), k.to(gpu), v.to(gpu), scale, input_pos, None, return_weights=True, return_lse=True)
    torch.cuda.synchronize()
    w_c = w.cpu()
    assert (w_c >= 0).all()
    torch.testing.assert_close(w_c.sum(-1), torch.full((B, Hkv), float(q_len)), rtol=5e-5, atol=3e-2)
    # oracle on KV head 3 (4 query heads)
    h = 3
    o_ref, w_ref = O.sdpa_in_blocks(q[:, 4 * h : 4 * h + 4], k[:, h : h + 1], v[:, h : h + 1], scale, input_pos, None)
    check_o(out.permute(0, 2, 1, 3)[:, 4 * h : 4 * h + 4], o_ref)
    torch.testing.assert_close(w_c[:, h : h + 1], w_ref, rtol=W_RTOL, atol=1e-6)
    # scattered layout: permute slots independently per head
    perm = torch.stack([torch.randperm(T, generator=gen) for _ in range(Hkv)]).view(B, Hkv, T)
    gi = perm.unsqueeze(-1).expand(-1, -1, -1, D)
    out_s, w_s, _ = ops.prefill_core(q.to(gpu), k.gather(2, gi).to(gpu), v.gather(2, gi).to(gpu), scale, input_pos,
                                     perm.to(torch.int32).to(gpu), return_weights=True)
    torch.cuda.synchronize()
    # same values, other summation order and other running maxima: equal up to bf16 rounding
    assert rel_err(out_s.float().cpu(), out.float().cpu()) < 1e-2
    w_back = torch.zeros_like(w_c).scatter_(-1, perm, w_s.cpu())
    torch.testing.assert_close(w_back, w_c, rtol=W_RTOL, atol=1e-6)


def _random_cases(n, seed):
    """Seeded shapes that mix what the fixed cases vary one at a time: group size, head size, ragged
    query and key counts, forced splits, position layout, store."""
    import random

    rnd = random.Random(seed)
    cases = []
    for _ in range(n):
        G = rnd.choice([1, 2, 3, 4, 5, 6, 7, 8])
        Hkv = rnd.choice([1, 2, 3])
        D = rnd.choice([64, 128])
        T = rnd.choice([1, 2, 63, 64, 65, 127, 200, 333, 512, 777, 1025, 2049])
        q_len = rnd.randint(1, min(T, 150))
        cases.append((len(cases), rnd.choice([1, 2]), G * Hkv, Hkv, q_len, T, D, rnd.choice([0, 0, 1, 2, 3, 5]), rnd.choice(["contig", "scattered"]),
                      rnd.choice(["bf16", "bf16", "u8", "u4"])))
    return cases


@pytest.mark.parametrize("case", _random_cases(28, 20240607), ids=lambda c: "-".join(str(x) for x in c))
def test_prefill_and_decode_random_shapes(gpu, case):
    n, B, Hq, Hkv, q_len, T, D, splits, layout, store = case
    q, k, v, gen = make_qkv(5000 + n, B, Hq, Hkv, q_len, T, D)
    scale = 1.0 / math.sqrt(D)
    if layout == "contig":
        input_pos, tp = T - q_len, None
    else:
        input_pos = T + 37
        tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    quant = None
    kg, vg = k.to(gpu), v.to(gpu)
    if store != "bf16":
        bits = 8 if store == "u8" else 4
        (kc, ks, kz), (vc, vs, vz) = O.quantize_rows(k, bits), O.quantize_rows(v, bits)
        k, v = O.dequantize_rows(kc, ks, kz), O.dequantize_rows(vc, vs, vz)
        if bits == 4:
            kc, vc = O.compress4(kc), O.compress4(vc)
        kg, vg = kc.to(gpu), vc.to(gpu)
        quant = ops.QuantState(ks.to(gpu), kz.to(gpu), vs.to(gpu), vz.to(gpu))
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, None if tp is None else tp.long())
    out, w, lse = ops.prefill_core(q.to(gpu), kg, vg, scale, input_pos, None if tp is None else tp.to(gpu), return_weights=True,
                                   return_lse=True, output_transposed=False, quant=quant, num_splits=splits)
    torch.cuda.synchronize()
    assert rel_err(out.float().cpu(), o_ref.float()) < 2e-2
    torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(lse.cpu(), O.lse2(q, k, scale, input_pos, None if tp is None else tp.long()), rtol=0, atol=2e-3)
    # single-token decode over the same store (unmasked: the new token is the newest)
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], k, v, scale, 10 * T + 100, None)
    out1, w1, _ = ops.decode_core(q[:, :, :1].to(gpu), kg, vg, scale, return_weights=True, quant=quant)
    torch.cuda.synchronize()
    assert rel_err(out1.float().cpu().unsqueeze(2), o1_ref.float()) < 2e-2
    torch.testing.assert_close(w1.cpu(), w1_ref, rtol=1e-3, atol=1e-6)


def _random_cases_wide(n, seed):
    """A second seeded mix over what later builds added: up to 16 heads per KV head, head size 256, float16 rows,
    quantised stores of every one of them."""
    import random

    rnd = random.Random(seed)
    cases = []
    for _ in range(n):
        D = rnd.choice([64, 128, 256])
        G = rnd.choice([1, 2, 4, 6, 8] if D == 256 else [1, 3, 4, 8, 9, 12, 16])
        Hkv = rnd.choice([1, 2])
        T = rnd.choice([3, 64, 97, 256, 511, 1000, 1537])
        q_len = rnd.randint(1, min(T, 100))
        cases.append((len(cases), rnd.choice([1, 2]), G * Hkv, Hkv, q_len, T, D, rnd.choice([0, 0, 2]), rnd.choice(["contig", "scattered"]),
                      rnd.choice(["plain", "u8", "u8", "u4"]), rnd.choice(["bf16", "f16"])))
    return cases


@pytest.mark.parametrize("case", _random_cases_wide(24, 77), ids=lambda c: "-".join(str(x) for x in c))
def test_prefill_and_decode_random_shapes_wide(gpu, case):
    n, B, Hq, Hkv, q_len, T, D, splits, layout, store, dt = case
    dtype = torch.bfloat16 if dt == "bf16" else torch.float16
    q, k, v, gen = make_qkv(9000 + n, B, Hq, Hkv, q_len, T, D, dtype=dtype)
    scale = 1.0 / math.sqrt(D)
    if layout == "contig":
        input_pos, tp = T - q_len, None
    else:
        input_pos = T + 37
        tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    quant = None
    kg, vg = k.to(gpu), v.to(gpu)
    if store != "plain":
        bits = 8 if store == "u8" else 4
        (kc, ks, kz), (vc, vs, vz) = O.quantize_rows(k, bits), O.quantize_rows(v, bits)
        k, v = O.dequantize_rows(kc, ks, kz, dtype), O.dequantize_rows(vc, vs, vz, dtype)
        if bits == 4:
            kc, vc = O.compress4(kc), O.compress4(vc)
        kg, vg = kc.to(gpu), vc.to(gpu)
        quant = ops.QuantState(ks.to(gpu), kz.to(gpu), vs.to(gpu), vz.to(gpu))
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, None if tp is None else tp.long())
    out, w, lse = ops.prefill_core(q.to(gpu), kg, vg, scale, input_pos, None if tp is None else tp.to(gpu), return_weights=True,
                                   return_lse=True, output_transposed=False, quant=quant, num_splits=splits)
    torch.cuda.synchronize()
    assert out.dtype == dtype
    assert rel_err(out.float().cpu(), o_ref.float()) < 2e-2
    torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    torch.testing.assert_close(lse.cpu(), O.lse2(q, k, scale, input_pos, None if tp is None else tp.long()), rtol=0, atol=2e-3)
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], k, v, scale, 10 * T + 100, None)
    out1, w1, _ = ops.decode_core(q[:, :, :1].to(gpu), kg, vg, scale, return_weights=True, quant=quant)
    torch.cuda.synchronize()
    assert rel_err(out1.float().cpu().unsqueeze(2), o1_ref.float()) < 2e-2
    torch.testing.assert_close(w1.cpu(), w1_ref, rtol=1e-3, atol=1e-6)


# ---- float16 queries / keys / values and head size 256 (keys_values/attention/flashinfer_wrapper.py:276,311-319) ----

TYPED_CASES = [
    # dtype, B, Hq, Hkv, q_len, T, D, input_pos, scattered, splits
    (torch.float16, 1, 8, 2, 128, 1024, 64, 896, True, 2),
    (torch.float16, 2, 8, 2, 100, 333, 128, 233, False, 3),
    (torch.float16, 1, 4, 4, 37, 700, 128, 1000, True, 0),
    (torch.float16, 1, 4, 2, 70, 300, 256, 400, True, 2),
    (torch.bfloat16, 1, 8, 2, 128, 1024, 256, 896, True, 0),
    (torch.bfloat16, 2, 4, 1, 33, 200, 256, 167, False, 1),
    (torch.bfloat16, 1, 4, 2, 300, 300, 256, 0, False, 2),  # square causal prefill
    (torch.float16, 1, 16, 2, 40, 900, 128, 1000, True, 0),  # 8 heads per KV head: the decode step multiplies on the matrix cores
    (torch.float16, 1, 16, 1, 20, 450, 64, 500, False, 0),
]


@pytest.mark.parametrize("dtype,B,Hq,Hkv,q_len,T,D,input_pos,scattered,splits", TYPED_CASES)
def test_prefill_decode_fp16_and_head_size_256(gpu, dtype, B, Hq, Hkv, q_len, T, D, input_pos, scattered, splits):
    q, k, v, gen = make_qkv(200 + T + q_len + D, B, Hq, Hkv, q_len, T, D, dtype=dtype)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len) if scattered else None
    if tp is None and input_pos != T - q_len:
        tp = (torch.arange(T, dtype=torch.int32) + (input_pos - (T - q_len))).view(1, 1, T).expand(B, Hkv, T).contiguous()
    scale = 1.0 / math.sqrt(D)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, None if tp is None else tp.to(torch.int64))
    l_ref = O.lse2(q, k, scale, input_pos, tp)
    out, w, lse = ops.prefill_core(q.to(gpu), k.to(gpu), v.to(gpu), scale, input_pos, None if tp is None else tp.to(gpu),
                                   return_weights=True, return_lse=True, output_transposed=False, num_splits=splits)
    torch.cuda.synchronize()
    assert out.dtype == dtype
    check_o(out, o_ref)
    torch.testing.assert_close(lse.cpu(), l_ref, rtol=1e-4, atol=1e-3)
    check_w(w, w_ref, q_len)
    # the score-sum kernel alone, fed the oracle's log-sum-exp
    w2 = ops.score_sum_core(q.to(gpu), k.to(gpu), l_ref.to(gpu), scale, input_pos, None if tp is None else tp.to(gpu))
    check_w(w2, w_ref, q_len)
    # one new token over the same cache
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], k, v, scale, 10 * T, None)
    out1, w1, lse1 = ops.decode_core(q[:, :, :1].to(gpu), k.to(gpu), v.to(gpu), scale, return_weights=True, return_lse=True)
    torch.cuda.synchronize()
    assert out1.dtype == dtype
    check_o(out1.unsqueeze(2), o1_ref)
    check_w(w1, w1_ref, 1)
    torch.testing.assert_close(lse1.cpu(), O.lse2(q[:, :, :1], k, scale, 10 * T, None), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("dtype,D", [(torch.float16, 128), (torch.bfloat16, 256), (torch.float16, 256)])
def test_h2o_cache_steps_fp16_and_head_size_256(gpu, dtype, D):
    """The cache object with float16 rows / heads of 256: prefill, chunk steps and a single-token step
    against the oracle (the slot write is a copy of 16-bit rows, the V-norm policy reads them as float16)."""
    from keys_values_amd.kvcache.h2o import H2OKVCache, KVCacheParams

    B, Hq, Hkv, L, chunk = 1, 4, 2, 256, 32
    gen = torch.Generator().manual_seed(D)
    total = L + 2 * chunk + 1
    qs = torch.randn(B, Hq, total, D, generator=gen).to(dtype)
    ks = torch.randn(B, Hkv, total, D, generator=gen).to(dtype)
    vs = torch.randn(B, Hkv, total, D, generator=gen).to(dtype)
    ref = O.H2OCacheOracle(B, Hq, Hkv, L, D, dtype=dtype, max_chunk_size=chunk)
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq, dtype), max_chunk_size=chunk, device=gpu)
    ref.prefill(qs[:, :, :L], ks[:, :, :L], vs[:, :, :L])
    cache.forward(qs[:, :, :L].to(gpu), ks[:, :, :L].to(gpu), vs[:, :, :L].to(gpu))
    pos = L
    for num in (chunk, chunk, 1):
        sl = slice(pos, pos + num)
        had = ref.next_index is not None
        o_ref, _, index = ref.forward(qs[:, :, sl], ks[:, :, sl], vs[:, :, sl])
        if had:
            cache.set_next_positions(index)
        o = cache.forward(qs[:, :, sl].to(gpu), ks[:, :, sl].to(gpu), vs[:, :, sl].to(gpu))
        torch.cuda.synchronize()
        assert o.dtype == dtype
        assert rel_err(o.float().cpu().view(B, num, Hq, D).transpose(1, 2), o_ref.float()) < 2e-2
        assert torch.equal(cache.k.cpu(), ref.k) and torch.equal(cache.v.cpu(), ref.v)
        assert torch.equal(cache.token_pos.cpu(), ref.token_pos)
        torch.testing.assert_close(cache.scores.cpu(), ref.scores, rtol=2e-3, atol=1e-5)
        pos += num


def test_gate_mirrors_the_reference(gpu):
    from keys_values_amd.attention.sdpa import can_do_hip_sdpa

    # keys_values/attention/flashinfer_wrapper.py:311-319: float16 or bfloat16, head sizes up to 256
    for dtype in (torch.float16, torch.bfloat16):
        for hs in (1, 48, 64, 100, 128, 200, 256):
            assert can_do_hip_sdpa(hs, dtype, True) and can_do_hip_sdpa(hs, dtype, False)
        assert not can_do_hip_sdpa(257, dtype)
    assert not can_do_hip_sdpa(128, torch.float32)
    # zero-padding from 129..255 to 256
    B, Hq, Hkv, q_len, T, D = 1, 4, 2, 9, 70, 200
    q, k, v, gen = make_qkv(43, B, Hq, Hkv, q_len, T, D, dtype=torch.float16)
    tp = scattered_positions(gen, B, Hkv, T, 100, q_len)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, 1 / math.sqrt(D), 100, tp.to(torch.int64))
    out, w = HipSDPA().scaled_dot_product_attention(q.to(gpu), k.to(gpu), v.to(gpu), None, 100, tp.to(gpu), return_attn_weights=True)
    assert out.shape == (B, Hq, q_len, D) and out.dtype == torch.float16
    check_o(out, o_ref)
    check_w(w, w_ref, q_len)


def test_decode_with_weights_beside_other_work(gpu):
    """The split kernel's wait for its row's other splits while another stream keeps the compute units busy
    (its workgroups then start at scattered times): same bits as on an idle device."""
    B, Hq, Hkv, T, D = 2, 8, 2, 30000, 128
    q, k, v, _ = make_qkv(4242, B, Hq, Hkv, 1, T, D)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    scale = 1.0 / math.sqrt(D)
    out0, w0, lse0 = ops.decode_core(qg, kg, vg, scale, return_weights=True, return_lse=True)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(gpu)
    busy = torch.randn(4096, 4096, device=gpu, dtype=torch.bfloat16)
    side.wait_stream(torch.cuda.current_stream(gpu))  # `busy` was made on the current stream
    for _ in range(3):
        with torch.cuda.stream(side):
            for _ in range(20):
                busy = (busy @ busy).clamp_(-1, 1)
        out1, w1, lse1 = ops.decode_core(qg, kg, vg, scale, return_weights=True, return_lse=True)
        torch.cuda.synchronize()
        assert torch.equal(out0, out1) and torch.equal(w0, w1) and torch.equal(lse0, lse1)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, T - 1, None)
    check_o(out0.unsqueeze(2), o_ref)
    check_w(w0, w_ref, 1)
