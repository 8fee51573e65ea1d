"""
The slot-structured prefill kernels (KVX_PREFILL_KERNEL=slots32 / slots64 in the environment: head size 128,
bf16 / fp16 rows; 64 rows per wavefront need at least 256 query rows per KV head, else 32 are used) against
the oracle, and against the default kernel on the same inputs.
"""
import math
import os

import pytest
import torch

from helpers import make_qkv, rel_err, scattered_positions
from keys_values_amd.attention import ops
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu

CASES = [
    # B, Hq, Hkv, q_len, T, input_pos, scattered, splits   (tile walks of 1, 2, 3, 5, 6 and 16 tiles, with and without splits)
    (1, 4, 1, 64, 64, 0, False, 1),
    (1, 4, 1, 64, 128, 64, False, 1),
    (1, 4, 1, 64, 192, 128, False, 1),
    (1, 8, 2, 100, 333, 233, False, 1),
    (1, 8, 2, 100, 333, 233, False, 3),
    (2, 8, 2, 128, 1024, 896, True, 2),
    (1, 8, 1, 37, 700, 1000, True, 0),
    (1, 4, 2, 300, 300, 0, False, 2),
    (2, 4, 4, 16, 200, 300, True, 1),       # fewer rows than a workgroup holds
]


@pytest.fixture(params=["slots32", "slots64"])
def variant(request):
    old = os.environ.get("KVX_PREFILL_KERNEL")
    os.environ["KVX_PREFILL_KERNEL"] = request.param
    yield request.param
    if old is None:
        del os.environ["KVX_PREFILL_KERNEL"]
    else:
        os.environ["KVX_PREFILL_KERNEL"] = old


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,q_len,T,input_pos,scattered,splits", CASES)
def test_slot_kernels_against_oracle(gpu, variant, B, Hq, Hkv, q_len, T, input_pos, scattered, splits, dtype):
    D = 128
    q, k, v, gen = make_qkv(300 + T + q_len, B, Hq, Hkv, q_len, T, D)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len) if scattered else None
    if tp is None and input_pos != T - q_len:
        tp = (torch.arange(T, dtype=torch.int32) + (input_pos - (T - q_len))).view(1, 1, T).expand(B, Hkv, T).contiguous()
    scale = 1.0 / math.sqrt(D)
    o_ref, w_ref = O.sdpa_in_blocks(q, k, v, scale, input_pos, None if tp is None else tp.to(torch.int64))
    l_ref = O.lse2(q, k, scale, input_pos, tp)
    args = (q.to(gpu), k.to(gpu), v.to(gpu), scale, input_pos, None if tp is None else tp.to(gpu))
    kw = dict(return_weights=True, return_lse=True, output_transposed=False, num_splits=splits)
    out, w, lse = ops.prefill_core(*args, **kw)
    torch.cuda.synchronize()
    # attention outputs within 2e-2 relative (measured: 3e-3 in bf16), log-sum-exp and score sums to fp32 accuracy
    assert rel_err(out.float().cpu(), o_ref.float()) < 6e-3
    torch.testing.assert_close(lse.cpu(), l_ref, rtol=1e-4, atol=1e-3)
    torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
    # the default kernel on the same inputs: same log-sum-exp to rounding, outputs equal to bf16 rounding
    os.environ["KVX_PREFILL_KERNEL"] = "classic"
    out32, w32, lse32 = ops.prefill_core(*args, **kw)
    os.environ["KVX_PREFILL_KERNEL"] = variant
    torch.cuda.synchronize()
    torch.testing.assert_close(lse, lse32, rtol=1e-5, atol=1e-4)
    assert rel_err(out.float(), out32.float()) < 6e-3
