"""GPU parity of quantised stores at head size 256 (rows spread over 32 lanes in the quantiser, four
wavefronts per workgroup in the chunk kernels, one workgroup per compute unit in the decode kernel) against
the CPU oracle, through the C ABI: the quantiser bit-exact, attention within the tolerances of the other
head sizes."""
import math

import pytest
import torch

from helpers import rel_err, scattered_positions
from keys_values_amd import _lib
from keys_values_amd.attention import ops
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu

D = 256


def rows_with_outliers(seed, rows, dtype):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, D, generator=gen)
    mask = torch.rand(rows, D, generator=gen) < 0.01
    x = torch.where(mask, torch.randn(rows, D, generator=gen) * 8, x).to(dtype)
    if rows >= 7:  # constant, all negative, tiny range, narrow range far from zero, one extreme per lane group
        x[0] = 0.0
        x[1] = -3.5
        x[2] = torch.linspace(-1e-3, 1e-3, D).to(dtype)
        x[3] = torch.linspace(100.0, 101.0, D).to(dtype)
        x[4, 255] = 1e4   # the maximum in the last of the row's 32 lanes
        x[5, 128] = -1e4  # the minimum in the first lane of the second half
    return x


def gpu_pack(kvx, x, bits, gpu):
    xg = x.reshape(-1, D).to(gpu)
    rows = xg.shape[0]
    c = torch.empty((rows, D * bits // 8), dtype=torch.uint8, device=gpu)
    s = torch.empty(rows, dtype=torch.float32, device=gpu)
    z = torch.empty(rows, dtype=torch.int32, device=gpu)
    _lib.check(kvx.kvx_quantize_rows_typed(xg.data_ptr(), D, rows, D, bits, _lib.elem_kv_dtype(x.dtype), c.data_ptr(), s.data_ptr(),
                                           z.data_ptr(), _lib.stream_ptr(gpu)))
    return c, s, z


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows", [1, 7, 1000, 70001])
def test_quantize_rows_256_bit_exact(kvx, gpu, bits, dtype, rows):
    x = rows_with_outliers(rows, rows, dtype)
    c_ref, s_ref, z_ref = O.quantize_rows(x, bits)
    c, s, z = gpu_pack(kvx, x, bits, gpu)
    out = torch.empty((rows, D), dtype=dtype, device=gpu)
    _lib.check(kvx.kvx_dequantize_rows_typed(c.data_ptr(), s.data_ptr(), z.data_ptr(), rows, D, bits, _lib.elem_kv_dtype(dtype), out.data_ptr(), D,
                                             _lib.stream_ptr(gpu)))
    torch.cuda.synchronize()
    assert torch.equal(s.cpu(), s_ref), "scales differ"
    assert torch.equal(z.cpu(), z_ref), "zero points differ"
    assert torch.equal(c.cpu(), O.compress4(c_ref) if bits == 4 else c_ref), "codes differ"
    assert torch.equal(out.cpu(), O.dequantize_rows(c_ref, s_ref, z_ref, dtype)), "dequantised rows differ"


@pytest.mark.parametrize("bits,dtype,B,Hq,Hkv,q_len,T", [
    (8, torch.bfloat16, 1, 8, 2, 96, 2048 + 40),   # 4 heads per KV head, a partial last tile
    (4, torch.bfloat16, 2, 4, 4, 33, 515),          # one head per KV head, ragged rows
    (8, torch.float16, 1, 8, 1, 150, 3000),         # 8 heads per KV head, more than one row block
    (4, torch.float16, 1, 6, 3, 64, 1100),          # 2 heads per KV head
    (8, torch.bfloat16, 1, 3, 1, 1, 9000),          # decode only, 3 heads padded to 4, several splits
])
def test_attention_over_quantised_cache_256(kvx, gpu, bits, dtype, B, Hq, Hkv, q_len, T):
    """Attention output and score-sums of a chunk (prefill kernel + score-sum kernel) and of a single token (decode
    kernel) over 8-bit and 4-bit stores of 256-value rows, dequantised inside the kernels, against the oracle run on
    the dequantised rows. Scattered token positions."""
    gen = torch.Generator().manual_seed(T + bits)
    k = rows_with_outliers(2, B * Hkv * T, dtype).view(B, Hkv, T, D)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(dtype)
    q = torch.randn(B, Hq, q_len, D, generator=gen).to(dtype)
    input_pos = T + 100
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len)
    kc, ks, kz = gpu_pack(kvx, k, bits, gpu)
    vc, vs, vz = gpu_pack(kvx, v, bits, gpu)
    W = D * bits // 8
    quant = ops.QuantState(ks.view(B, Hkv, T), kz.view(B, Hkv, T), vs.view(B, Hkv, T), vz.view(B, Hkv, T))
    kc, vc = kc.view(B, Hkv, T, W), vc.view(B, Hkv, T, W)
    kd = O.dequantize_rows(*O.quantize_rows(k, bits), dtype)
    vd = O.dequantize_rows(*O.quantize_rows(v, bits), dtype)
    scale = 1 / math.sqrt(D)
    if q_len > 1:
        o_ref, w_ref = O.sdpa_in_blocks(q, kd, vd, scale, input_pos, tp.long())
        out, w, _ = ops.prefill_core(q.to(gpu), kc, vc, scale, input_pos, tp.to(gpu), return_weights=True, quant=quant, output_transposed=False)
        torch.cuda.synchronize()
        assert out.dtype == dtype
        assert rel_err(out.float().cpu(), o_ref.float()) < 2e-2
        torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    o1_ref, w1_ref = O.sdpa_in_blocks(q[:, :, :1], kd, vd, scale, 10 * T, None)
    out1, w1, _ = ops.decode_core(q[:, :, :1].to(gpu), kc, vc, scale, return_weights=True, quant=quant)
    torch.cuda.synchronize()
    assert rel_err(out1.float().cpu().unsqueeze(2), o1_ref.float()) < 2e-2
    torch.testing.assert_close(w1.cpu(), w1_ref, rtol=1e-3, atol=1e-6)
