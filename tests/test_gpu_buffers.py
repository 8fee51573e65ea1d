"""The K/V buffer objects (the reference's KVCacheBuffers surface) and the KeysAndValues holders, driven
the way the reference's AttnWeightsKVCache drives its buffers: the cache logic here is the CPU oracle's,
only rows and attention run on the device."""
import math

import pytest
import torch

from helpers import rel_err
from keys_values_amd.attention import HipMultiHeadSelfAttention
from keys_values_amd.kvcache import (DefaultKeysAndValues, KVCacheBuffersParams, QuantizedKeysAndValues, create_kv_cache_buffers)
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("store,bits", [("default", None), ("torch-quantized8", 8), ("torch-quantized4", 4)])
def test_buffers_follow_the_oracles_slot_sequence(gpu, store, bits):
    """prefill, forward(positions, key, value) with the slots the oracle's H2O cache chooses, attention over
    the returned holder with the oracle's token positions: outputs and score-sums against the oracle, the
    buffers' content against the oracle's rows after every step."""
    B, Hq, Hkv, L, D, chunk = 2, 8, 2, 320, 64, 32
    gen = torch.Generator().manual_seed(21)
    total = L + 4 * chunk + 1
    qs = torch.randn(B, Hq, total, D, generator=gen).to(torch.bfloat16)
    ks = torch.randn(B, Hkv, total, D, generator=gen).to(torch.bfloat16)
    vs = torch.randn(B, Hkv, total, D, generator=gen).to(torch.bfloat16)
    stored = (lambda x: O.dequantize_rows(*O.quantize_rows(x, bits))) if bits else (lambda x: x)
    ref = O.H2OCacheOracle(B, Hq, Hkv, L, D, dtype=torch.bfloat16, max_chunk_size=chunk)
    bufs = create_kv_cache_buffers(store, KVCacheBuffersParams(B + 1, Hkv, D, None, torch.bfloat16), L)
    assert not bufs.buffers_are_allocated and bufs.get_keys_values() is None
    mha = HipMultiHeadSelfAttention()
    n0 = L - chunk  # the first step after the prefill fills the cache
    ref.prefill(qs[:, :, :n0], ks[:, :, :n0], vs[:, :, :n0], stored(ks[:, :, :n0]), stored(vs[:, :, :n0]))
    bufs.prefill(ks[:, :, :n0].to(gpu), vs[:, :, :n0].to(gpu))
    assert bufs.buffers_are_allocated and bufs.device == gpu and bufs.batch_size == B and bufs.current_length == n0
    # the first chunk attends over what it is given (keys_values/kvcache/base.py:567-571)
    o0, w0 = mha(qs[:, :, :n0].to(gpu), DefaultKeysAndValues(ks[:, :, :n0].to(gpu), vs[:, :, :n0].to(gpu)), input_pos=0)
    o0_ref, _ = O.sdpa_in_blocks(qs[:, :, :n0], ks[:, :, :n0], vs[:, :, :n0], 1 / math.sqrt(D), 0, None, return_attn_weights=False)
    assert w0 is None and rel_err(o0.float().cpu().view(B, n0, Hq, D).transpose(1, 2), o0_ref.float()) < 2e-2
    pos = n0
    for num in (chunk, chunk, 1, chunk, chunk):
        sl = slice(pos, pos + num)
        input_pos = ref.input_pos
        o_ref, w_ref, index = ref.forward(qs[:, :, sl], stored(ks[:, :, sl]), stored(vs[:, :, sl]))
        kv = bufs.forward(index.to(gpu), ks[:, :, sl].to(gpu), vs[:, :, sl].to(gpu))
        assert bufs.current_length == ref.current_length
        assert isinstance(kv, QuantizedKeysAndValues if bits else DefaultKeysAndValues)
        T = ref.current_length
        assert torch.equal(kv.keys().cpu(), ref.k[:, :, :T]) and torch.equal(kv.values().cpu(), ref.v[:, :, :T])
        o, w = mha(qs[:, :, sl].to(gpu), kv, input_pos=input_pos, return_attn_weights=True, token_positions=ref.token_pos[:, :, :T].to(gpu))
        assert o.shape == (B, num, Hq * D)
        assert rel_err(o.float().cpu().view(B, num, Hq, D).transpose(1, 2), o_ref.float()) < 2e-2
        torch.testing.assert_close(w.cpu(), w_ref, rtol=1e-3, atol=1e-6)
        gk, gv = bufs.get_slots(index.to(gpu))
        assert torch.equal(gk.cpu(), stored(ks[:, :, sl])) and torch.equal(gv.cpu(), stored(vs[:, :, sl]))
        pos += num
    # ranges, the whole view, sizes, deallocation
    rk, rv = bufs.get_slots((5, 9))
    assert torch.equal(rk.cpu(), ref.k[:, :, 5:9]) and torch.equal(rv.cpu(), ref.v[:, :, 5:9])
    bufs.set_slots((5, 9), ks[:, :, :4].to(gpu), vs[:, :, :4].to(gpu))
    rk, _ = bufs.get_slots((5, 9))
    assert torch.equal(rk.cpu(), stored(ks[:, :, :4]))
    bufs.write_back()
    total_bits, parts = bufs.size_estimate()
    apriori, _ = type(bufs).size_estimate_apriori(bufs.get_params(), cache_length=L, num_bits=bits)
    assert total_bits == sum(parts.values()) and apriori == total_bits * (B + 1) // bufs.k.shape[0]
    with pytest.raises(ValueError):
        bufs.set_slots((0, 3), ks[:, :, :4].to(gpu), vs[:, :, :4].to(gpu))
    with pytest.raises(ValueError):
        bufs.prefill(ks[:, :1, :4].to(gpu), vs[:, :1, :4].to(gpu))
    bufs.deallocate()
    assert not bufs.buffers_are_allocated and bufs.current_length == 0
    with pytest.raises(IndexError):
        bufs.get_slots((0, 1))


def test_buffers_reject_the_cpu(gpu):
    bufs = create_kv_cache_buffers("default", KVCacheBuffersParams(1, 2, 64, None, torch.bfloat16), 16)
    with pytest.raises(RuntimeError):
        bufs.prefill(torch.zeros(1, 2, 4, 64, dtype=torch.bfloat16), torch.zeros(1, 2, 4, 64, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        create_kv_cache_buffers("bnb-quantized4", KVCacheBuffersParams(1, 2, 64, None, torch.bfloat16), 16)


def test_buffers_before_prefill_raise_a_clear_error(gpu):
    """forward / set_slots / get_slots on buffers that have not seen a prefill: IndexError, not a TypeError from None."""
    bufs = create_kv_cache_buffers("default", KVCacheBuffersParams(1, 2, 64, None, torch.bfloat16), 16)
    x = torch.zeros(1, 2, 4, 64, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(IndexError):
        bufs.forward((0, 4), x, x)
    with pytest.raises(IndexError):
        bufs.set_slots((0, 4), x, x)
    with pytest.raises(IndexError):
        bufs.get_slots((0, 4))
