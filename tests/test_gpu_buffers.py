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


def _oracle_blocks(x, bits):
    """Codes, scales and zero points of the slots of x (B, Hkv, n, D), one block per slot over the heads."""
    return O.quantize_store(x, bits, True)


@pytest.mark.parametrize("bits,dtype", [(8, torch.bfloat16), (4, torch.bfloat16), (8, torch.float16)])
def test_buffers_with_blocks_over_heads(gpu, bits, dtype):
    """The store whose quantisation blocks run over the heads (keys_values/kvcache/quant_buffers.py:849-870),
    through the buffer interface: a prefill leaves what the reference's quantiser leaves
    (keys_values/kvcache/quantize/pytorch.py:235-245,312-355); a write to slots that differ per head requantises each
    touched slot from the new rows and the dequantised rows of the other heads, which is what the reference's
    write-back of its dequantised working buffer does to it (keys_values/kvcache/quant_buffers.py:368-375); reads
    return the dequantised rows. Bit-exact against the oracle."""
    B, Hkv, L, D, num = 2, 4, 96, 64, 5
    gen = torch.Generator().manual_seed(bits)
    params = KVCacheBuffersParams(B, Hkv, D, gpu, dtype)
    buf = create_kv_cache_buffers(f"torch-quantized{bits}", params, L, blocks_over_heads=True)
    assert buf.blocks_over_heads
    k0 = torch.randn(B, Hkv, L, D, generator=gen).to(dtype)
    v0 = (torch.randn(B, Hkv, L, D, generator=gen) * 3).to(dtype)
    buf.prefill(k0.to(gpu), v0.to(gpu))
    shape = (B, Hkv, L, D)
    state = {}
    for name, x, codes, sc, zp in (("k", k0, buf.k, buf.k_scale, buf.k_zp), ("v", v0, buf.v, buf.v_scale, buf.v_zp)):
        c_ref, s_ref, z_ref = _oracle_blocks(x, bits)
        assert tuple(codes.shape) == (B, L, Hkv * D * bits // 8) and tuple(sc.shape) == (B, L)
        assert torch.equal(codes.cpu(), c_ref) and torch.equal(sc.cpu(), s_ref) and torch.equal(zp.cpu(), z_ref), name
        state[name] = O.dequantize_store(c_ref, s_ref, z_ref, shape, bits, True, dtype).contiguous()
        state[name + "_codes"] = (c_ref, s_ref, z_ref)
    kv = buf.get_keys_values()
    assert torch.equal(kv.keys().cpu(), state["k"]) and torch.equal(kv.values().cpu(), state["v"])
    # slots that differ per head (and overlap between heads), two rounds
    for rnd in range(2):
        pos = torch.stack([torch.stack([torch.randperm(L, generator=gen)[:num] for _ in range(Hkv)]) for _ in range(B)]).to(torch.int32)
        old, shared = pos[0, 1, 0].item(), pos[0, 0, 0].item()  # two heads write the same slot
        pos[0, 1][pos[0, 1] == shared] = old
        pos[0, 1, 0] = shared
        k1 = torch.randn(B, Hkv, num, D, generator=gen).to(dtype)
        v1 = torch.randn(B, Hkv, num, D, generator=gen).to(dtype)
        buf.set_slots(pos.to(gpu), k1.to(gpu), v1.to(gpu))
        for name, new, codes, sc, zp in (("k", k1, buf.k, buf.k_scale, buf.k_zp), ("v", v1, buf.v, buf.v_scale, buf.v_zp)):
            work = state[name].clone()  # the dequantised working buffer
            gi = pos.long().unsqueeze(-1).expand(-1, -1, -1, D)
            work.scatter_(2, gi, new)
            touched = torch.zeros(B, L, dtype=torch.bool)
            for b in range(B):
                touched[b, pos[b].reshape(-1).long()] = True
            c_all, s_all, z_all = _oracle_blocks(work, bits)
            got_c, got_s, got_z = codes.cpu(), sc.cpu(), zp.cpu()
            assert torch.equal(got_c[touched], c_all[touched]) and torch.equal(got_s[touched], s_all[touched]) and torch.equal(got_z[touched], z_all[touched])
            # untouched slots keep their codes: nothing else was requantised
            old_c, old_s, old_z = state[name + "_codes"]
            assert torch.equal(got_c[~touched], old_c[~touched]) and torch.equal(got_s[~touched], old_s[~touched]) and torch.equal(got_z[~touched], old_z[~touched])
            state[name + "_codes"] = (got_c, got_s, got_z)
            state[name] = O.dequantize_store(got_c, got_s, got_z, shape, bits, True, dtype).contiguous()
        kk, vv = buf.get_slots(pos.to(gpu))
        gi = pos.long().unsqueeze(-1).expand(-1, -1, -1, D)
        assert torch.equal(kk.cpu(), state["k"].gather(2, gi)) and torch.equal(vv.cpu(), state["v"].gather(2, gi))
        kk, vv = buf.get_slots((7, 19))
        assert torch.equal(kk.cpu(), state["k"][:, :, 7:19]) and torch.equal(vv.cpu(), state["v"][:, :, 7:19])
    # a range write replaces whole blocks
    k2 = torch.randn(B, Hkv, 8, D, generator=gen).to(dtype)
    buf.set_slots((16, 24), k2.to(gpu), k2.to(gpu))
    c_ref, s_ref, z_ref = _oracle_blocks(k2, bits)
    assert torch.equal(buf.k[:, 16:24].cpu(), c_ref) and torch.equal(buf.v_scale[:, 16:24].cpu(), s_ref)
