"""GPU parity of the 4-bit store and of quantisation blocks that run over the heads, against the CPU
oracle (bit-exact), through the C ABI."""
import ctypes

import pytest
import torch

from keys_values_amd import _lib
from keys_values_amd.kvcache.quantize import RowQuantizer
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu


def outlier_rows(seed, rows, D):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, D, generator=gen)
    mask = torch.rand(rows, D, generator=gen) < 0.01
    x = torch.where(mask, torch.randn(rows, D, generator=gen) * 8, x).to(torch.bfloat16)
    if rows >= 7:  # constant, all negative, tiny range, wide range, extremes of the bf16 dynamics
        x[0] = 0.0
        x[1] = -3.5
        x[2] = torch.linspace(-1e-3, 1e-3, D).to(torch.bfloat16)
        x[3] = torch.linspace(100.0, 101.0, D).to(torch.bfloat16)
        x[4] = 7.0
        x[5, ::2] = -1e4
    return x


@pytest.mark.parametrize("rows,D", [(1, 128), (7, 64), (1000, 128), (4099, 64), (65536, 128), (8 * 65536, 128)])
def test_quantize_rows4_bit_exact(kvx, gpu, rows, D):
    x = outlier_rows(rows, rows, D)
    c_ref, s_ref, z_ref = O.quantize_rows(x, num_bits=4)
    p_ref = O.compress4(c_ref)
    xg = x.to(gpu)
    packed = torch.empty((rows, D // 2), dtype=torch.uint8, device=gpu)
    sc = torch.empty(rows, dtype=torch.float32, device=gpu)
    zp = torch.empty(rows, dtype=torch.int32, device=gpu)
    st = _lib.stream_ptr(gpu)
    _lib.check(kvx.kvx_quantize_rows4(xg.data_ptr(), D, rows, D, packed.data_ptr(), sc.data_ptr(), zp.data_ptr(), st))
    out = torch.empty((rows, D), dtype=torch.bfloat16, device=gpu)
    _lib.check(kvx.kvx_dequantize_rows4(packed.data_ptr(), sc.data_ptr(), zp.data_ptr(), rows, D, out.data_ptr(), D, st))
    torch.cuda.synchronize()
    assert torch.equal(sc.cpu(), s_ref), "scales differ"
    assert torch.equal(zp.cpu(), z_ref), "zero points differ"
    assert torch.equal(packed.cpu(), p_ref), "packed codes differ"
    assert torch.equal(out.cpu(), O.dequantize_rows(c_ref, s_ref, z_ref, torch.bfloat16)), "dequantised rows differ"


def test_quantize_rows4_empty_and_bad_arguments(kvx, gpu):
    assert kvx.kvx_quantize_rows4(None, 128, 0, 128, None, None, None, None) == 0
    assert kvx.kvx_quantize_rows4(None, 100, 4, 100, None, None, None, None) == _lib.KVX_ERR_UNSUPPORTED
    a = _lib.BlockQuantArgs()
    a.n_outer, a.n_inner, a.nseg, a.D, a.bits = 1, 1, 1, 64, 3
    assert kvx.kvx_quantize_blocks(ctypes.byref(a), None) == _lib.KVX_ERR_UNSUPPORTED and b"bits" in kvx.kvx_last_error()
    a.bits, a.nseg, a.D = 4, 128, 128  # 16384 values per block
    assert kvx.kvx_quantize_blocks(ctypes.byref(a), None) == _lib.KVX_ERR_UNSUPPORTED


@pytest.mark.parametrize("num_bits", [4, 8])
@pytest.mark.parametrize("blocks_over_heads", [False, True])
@pytest.mark.parametrize("shape", [(3, 4, 32, 64), (2, 8, 100, 128), (1, 5, 17, 48)])
def test_store_matches_oracle_and_known_answer(gpu, num_bits, blocks_over_heads, shape):
    """The quantiser surface (quantize / dequantize over slot ranges, quantization_error) against the
    oracle's store, bit for bit; and test/kvcache/test_quantization.py:647-766: integers holding both
    extremes in every head row survive the round trip exactly."""
    B, Hkv, L, D = shape
    qz = RowQuantizer(shape, torch.bfloat16, num_bits, blocks_over_heads, allocate_buffers=True, device=gpu)
    first, final = (B, Hkv * D) if blocks_over_heads else (B * Hkv, D)
    assert qz.quant_buffer.shape == (first, L, final * num_bits // 8) and qz.quant_buffer.dtype == torch.uint8
    assert qz.quant_scales.shape == (first, L) and qz.quant_zero_points.dtype == torch.int32
    x = outlier_rows(L, B * Hkv * L, D).view(B, Hkv, L, D)
    qz.quantize(0, L, x.to(gpu))
    buf, s, z = O.quantize_store(x, num_bits, blocks_over_heads)
    assert torch.equal(qz.quant_scales.cpu(), s) and torch.equal(qz.quant_zero_points.cpu(), z)
    assert torch.equal(qz.quant_buffer.cpu(), buf)
    assert torch.equal(qz.dequantize(0, L).cpu(), O.dequantize_store(buf, s, z, shape, num_bits, blocks_over_heads))
    # a slot range, from a strided view, leaves the other slots alone
    lo, hi = 3, min(L, 3 + 9)
    y = outlier_rows(7, B * Hkv * L * 2, D).view(B, Hkv, L * 2, D).to(gpu)[:, :, : 2 * (hi - lo) : 2]
    qz.quantize(lo, hi, y)
    buf2, s2, z2 = O.quantize_store(y.cpu(), num_bits, blocks_over_heads)
    assert torch.equal(qz.quant_buffer[:, lo:hi].cpu(), buf2) and torch.equal(qz.quant_scales[:, lo:hi].cpu(), s2)
    assert torch.equal(qz.quant_zero_points[:, lo:hi].cpu(), z2)
    assert torch.equal(qz.quant_buffer[:, :lo].cpu(), buf[:, :lo]) and torch.equal(qz.quant_buffer[:, hi:].cpu(), buf[:, hi:])
    part = qz.dequantize(lo, hi)
    assert torch.equal(part.cpu(), O.dequantize_store(buf2, s2, z2, (B, Hkv, hi - lo, D), num_bits, blocks_over_heads))
    # quantisation error
    if not blocks_over_heads:
        torch.testing.assert_close(qz.quantization_error(y).cpu(), O.quantization_error(y.cpu(), num_bits), rtol=1e-5, atol=1e-6)
    # known answer
    gen = torch.Generator().manual_seed(31415927)
    high = 2**num_bits
    data = torch.randint(0, high, shape, generator=gen)
    i0 = torch.randint(0, D, shape[:-1], generator=gen)
    i1 = (i0 + 1 + torch.randint(0, D - 1, shape[:-1], generator=gen)) % D
    data.scatter_(-1, i0.unsqueeze(-1), 0)
    data.scatter_(-1, i1.unsqueeze(-1), high - 1)
    xi = data.to(torch.bfloat16).to(gpu)
    qz.quantize(0, L, xi)
    assert torch.equal(qz.dequantize(0, L), xi)
    codes = qz.quant_buffer.cpu()
    codes = O.uncompress4(codes) if num_bits == 4 else codes
    want = data.transpose(1, 2).reshape(B, L, Hkv * D) if blocks_over_heads else data.reshape(B * Hkv, L, D)
    assert torch.equal(codes.long(), want)


def test_blocks_over_heads_store_feeds_attention(gpu):
    """An 8-bit store whose blocks run over the heads is read by the attention kernels as it is: the
    codes are (B, L, Hkv, D) by strides and all heads of a token share one scale / zero point."""
    import math

    from keys_values_amd.attention import ops
    from helpers import rel_err

    B, Hq, Hkv, L, D, q_len = 2, 8, 4, 700, 128, 40
    gen = torch.Generator().manual_seed(1)
    k = torch.randn(B, Hkv, L, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, Hkv, L, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, Hq, q_len, D, generator=gen).to(torch.bfloat16)
    qk = RowQuantizer((B, Hkv, L, D), torch.bfloat16, 8, True, allocate_buffers=True, device=gpu)
    qv = RowQuantizer((B, Hkv, L, D), torch.bfloat16, 8, True, allocate_buffers=True, device=gpu)
    qk.quantize(0, L, k.to(gpu))
    qv.quantize(0, L, v.to(gpu))
    kc = qk.quant_buffer.view(B, L, Hkv, D).permute(0, 2, 1, 3)
    vc = qv.quant_buffer.view(B, L, Hkv, D).permute(0, 2, 1, 3)
    shared = lambda t: t.view(B, 1, L).expand(B, Hkv, L)  # noqa: E731  head stride 0
    quant = ops.QuantState(shared(qk.quant_scales), shared(qk.quant_zero_points), shared(qv.quant_scales), shared(qv.quant_zero_points))
    kd = O.dequantize_store(*O.quantize_store(k, 8, True), (B, Hkv, L, D), 8, True)
    vd = O.dequantize_store(*O.quantize_store(v, 8, True), (B, Hkv, L, D), 8, True)
    scale = 1 / math.sqrt(D)
    o_ref, w_ref = O.sdpa_in_blocks(q, kd, vd, scale, L - q_len, None)
    out, w, _ = ops.prefill_core(q.to(gpu), kc, vc, scale, L - q_len, None, return_weights=True, quant=quant, output_transposed=False)
    torch.cuda.synchronize()
    assert rel_err(out.float().cpu(), o_ref.float()) < 2e-2
    torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], kd, vd, scale, L - 1, None)
    out1, w1, _ = ops.decode_core(q[:, :, :1].to(gpu), kc, vc, scale, return_weights=True, quant=quant)
    torch.cuda.synchronize()
    assert rel_err(out1.float().cpu().unsqueeze(2), o1_ref.float()) < 2e-2
    torch.testing.assert_close(w1.cpu(), w1_ref, rtol=1e-3, atol=1e-6)


@pytest.mark.parametrize("B,Hq,Hkv,q_len,T,D", [(1, 8, 2, 96, 2048 + 40, 128), (2, 4, 4, 33, 515, 64), (1, 8, 1, 1, 3000, 128),
                                                 (1, 16, 1, 1, 1500, 64), (2, 8, 4, 1, 4100, 128)])
def test_attention_over_4bit_cache(kvx, gpu, B, Hq, Hkv, q_len, T, D):
    """Attention output, score-sums (prefill kernel + score-sum kernel) and single-token decode over the
    4-bit store, the nibbles unpacked and dequantised inside the kernels, against the oracle run on
    the dequantised bf16 rows. Scattered token positions."""
    import math

    from helpers import rel_err, scattered_positions
    from keys_values_amd.attention import ops

    gen = torch.Generator().manual_seed(T)
    k = outlier_rows(2, B * Hkv * T, D).view(B, Hkv, T, D)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, Hq, q_len, D, generator=gen).to(torch.bfloat16)
    input_pos = T + 100
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    st = _lib.stream_ptr(gpu)

    def pack(x):
        xg = x.reshape(-1, D).to(gpu)
        rows = xg.shape[0]
        c = torch.empty((rows, D // 2), dtype=torch.uint8, device=gpu)
        s = torch.empty(rows, dtype=torch.float32, device=gpu)
        z = torch.empty(rows, dtype=torch.int32, device=gpu)
        _lib.check(kvx.kvx_quantize_rows4(xg.data_ptr(), D, rows, D, c.data_ptr(), s.data_ptr(), z.data_ptr(), st))
        return c.view(B, Hkv, T, D // 2), s.view(B, Hkv, T), z.view(B, Hkv, T)

    kc, ks, kz = pack(k)
    vc, vs, vz = pack(v)
    quant = ops.QuantState(ks, kz, vs, vz)
    kd = O.dequantize_rows(*O.quantize_rows(k, 4))
    vd = O.dequantize_rows(*O.quantize_rows(v, 4))
    scale = 1 / math.sqrt(D)
    if q_len > 1:
        o_ref, w_ref = O.sdpa_in_blocks(q, kd, vd, scale, input_pos, tp.long())
        out, w, _ = ops.prefill_core(q.to(gpu), kc, vc, scale, input_pos, tp.to(gpu), return_weights=True, quant=quant,
                                     output_transposed=False)
        torch.cuda.synchronize()
        assert rel_err(out.float().cpu(), o_ref.float()) < 2e-2
        torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], kd, vd, scale, 10 * T, None)
    out1, w1, _ = ops.decode_core(q[:, :, :1].to(gpu), kc, vc, scale, return_weights=True, quant=quant)
    torch.cuda.synchronize()
    assert rel_err(out1.float().cpu().unsqueeze(2), o1_ref.float()) < 2e-2
    torch.testing.assert_close(w1.cpu(), w1_ref, rtol=1e-3, atol=1e-6)
