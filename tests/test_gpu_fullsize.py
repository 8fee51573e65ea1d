"""The benchmark configurations at their real sizes, where KV splits, 32-bit tile offsets, 8-wavefront
workgroups and offsets beyond 2^31 all matter: quantised chunked prefill at 65536 slots against the
oracle, the Qwen3-4B-shaped stack at real widths (properties), 256 decode steps over 8 x 131072
slots (properties + one row against the oracle), and bit-reproducibility of every kernel family."""
import ctypes
import math

import pytest
import torch

from helpers import rel_err, scattered_positions
from keys_values_amd import _lib
from keys_values_amd.attention import ops
from keys_values_amd.kvcache.h2o import H2OKVCache, KVCacheParams
from oracle import kvx_oracle as O

pytestmark = pytest.mark.gpu


def _quantize_store(kvx, gpu, x, bits):
    """x (B, Hkv, T, D) bf16 on the device -> codes (B, Hkv, T, D or D/2) uint8, scale, zp (B, Hkv, T)."""
    B, Hkv, T, D = x.shape
    rows = B * Hkv * T
    codes = torch.empty((rows, D if bits == 8 else D // 2), dtype=torch.uint8, device=gpu)
    sc = torch.empty(rows, dtype=torch.float32, device=gpu)
    zp = torch.empty(rows, dtype=torch.int32, device=gpu)
    fn = kvx.kvx_quantize_rows if bits == 8 else kvx.kvx_quantize_rows4
    _lib.check(fn(x.data_ptr(), D, rows, D, codes.data_ptr(), sc.data_ptr(), zp.data_ptr(), _lib.stream_ptr(gpu)))
    return codes.view(B, Hkv, T, -1), sc.view(B, Hkv, T), zp.view(B, Hkv, T)


def _dequantize_store(kvx, gpu, codes, sc, zp, D, bits):
    B, Hkv, T, _ = codes.shape
    out = torch.empty((B, Hkv, T, D), dtype=torch.bfloat16, device=gpu)
    fn = kvx.kvx_dequantize_rows if bits == 8 else kvx.kvx_dequantize_rows4
    _lib.check(fn(codes.data_ptr(), sc.data_ptr(), zp.data_ptr(), B * Hkv * T, D, out.data_ptr(), D, _lib.stream_ptr(gpu)))
    return out


@pytest.mark.parametrize("bits", [8, 4])
def test_quantised_prefill_at_65536_slots(kvx, gpu, bits):
    """B1, 32/8 heads, D128, 65536 slots, 1024 queries over the 8-bit and the 4-bit store: keys with 1 %
    outliers of 8 sigma, quantised on the device. The last KV head (largest offsets) against the oracle
    run on the dequantised rows; every row of score-sums adds up to the number of queries; and the
    kernels that dequantise on load give what the bf16 kernels give on the dequantised copy."""
    B, Hq, Hkv, q_len, T, D = 1, 32, 8, 1024, 65536, 128
    G = Hq // Hkv
    gen = torch.Generator().manual_seed(2)
    k = torch.randn(B, Hkv, T, D, generator=gen)
    mask = torch.rand(B, Hkv, T, D, generator=gen) < 0.01
    k = torch.where(mask, torch.randn(B, Hkv, T, D, generator=gen) * 8, k).to(torch.bfloat16)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16)
    q = torch.randn(B, Hq, q_len, D, generator=gen).to(torch.bfloat16)
    input_pos, scale = T - q_len, 1.0 / math.sqrt(D)
    print(f"quantised prefill bits={bits} T={T} q={q_len}", flush=True)
    kc, ks, kz = _quantize_store(kvx, gpu, k.to(gpu), bits)
    vc, vs, vz = _quantize_store(kvx, gpu, v.to(gpu), bits)
    quant = ops.QuantState(ks, kz, vs, vz)
    qg = q.to(gpu)
    out, w, lse = ops.prefill_core(qg, kc, vc, scale, input_pos, None, return_weights=True, return_lse=True, output_transposed=False, quant=quant)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and (w >= 0).all()
    torch.testing.assert_close(w.sum(-1), torch.full((B, Hkv), float(q_len), device=gpu), rtol=2e-4, atol=0)
    # the same values through the bf16 kernels
    kd = _dequantize_store(kvx, gpu, kc, ks, kz, D, bits)
    vd = _dequantize_store(kvx, gpu, vc, vs, vz, D, bits)
    out2, w2, lse2 = ops.prefill_core(qg, kd, vd, scale, input_pos, None, return_weights=True, return_lse=True, output_transposed=False)
    torch.cuda.synchronize()
    assert rel_err(out.float(), out2.float()) < 2e-3
    torch.testing.assert_close(lse, lse2, rtol=0, atol=1e-4)
    torch.testing.assert_close(w, w2, rtol=1e-4, atol=1e-7)
    # oracle on the last KV head, fed the rows as the CPU quantiser restatement leaves them
    h = Hkv - 1
    kq = O.quantize_rows(k[:, h : h + 1], bits)
    vq = O.quantize_rows(v[:, h : h + 1], bits)
    assert torch.equal(ks[:, h : h + 1].cpu(), kq[1]) and torch.equal(kz[:, h : h + 1].cpu(), kq[2])
    k_ref, v_ref = O.dequantize_rows(*kq), O.dequantize_rows(*vq)
    assert torch.equal(kd[:, h : h + 1].cpu(), k_ref) and torch.equal(vd[:, h : h + 1].cpu(), v_ref)
    qh = q[:, G * h : G * h + G]
    o_ref, w_ref = O.sdpa_in_blocks(qh, k_ref, v_ref, scale, input_pos, None)
    assert rel_err(out[:, G * h : G * h + G].float().cpu(), o_ref.float()) < 2e-2
    torch.testing.assert_close(w[:, h : h + 1].cpu(), w_ref, rtol=1e-3, atol=1e-6)
    lse_ref = O.lse2(qh, k_ref, scale, input_pos, None)
    torch.testing.assert_close(lse[:, :, G * h : G * h + G].cpu(), lse_ref, rtol=0, atol=1e-3)


def test_qwen3_4b_widths_two_layers_chunked_prefill(gpu):
    """The long-context configuration at its real widths (2560 hidden, 32/8 heads of 128, SwiGLU 9728,
    vocabulary 151936, cache of 16384 slots, chunks of 1024, 8-bit store), cut to two layers: the
    prefill chunk, the chunk under the initial rule and two H2O chunks. Checked: the chunk schedule,
    finite hidden states, per layer the score-sums of a chunk add up to its 1024 queries, and the slot
    bookkeeping (the slots announced by next_positions hold the chunk's positions in order, every other
    slot keeps its token, all positions of a row are distinct)."""
    from dataclasses import replace

    from keys_values_amd.longctx.model import QWEN3_4B, LongContextPrefillModel

    cfg = replace(QWEN3_4B, n_layer=2)
    L, chunk, B = 16384, 1024, 1
    model = LongContextPrefillModel(cfg, cache_length=L, chunk_size=chunk, max_batch_size=B, quantized=True, max_context=L + 4 * chunk, seed=4, device=gpu)
    ids = torch.randint(0, cfg.vocab_size, (B, L + 3 * chunk), generator=torch.Generator().manual_seed(4)).to(gpu)
    sizes = model.chunk_sizes(ids.shape[1])
    assert sizes == [L, chunk, chunk, chunk]
    w_sums = [[] for _ in model.caches]
    for li, cache in enumerate(model.caches):
        inner = cache._update

        def spy(attn_weights, query_length, inner=inner, li=li):
            w_sums[li].append(attn_weights.sum(-1))
            return inner(attn_weights, query_length)

        cache._update = spy
    model.reset()
    start = 0
    for ci, n in enumerate(sizes):
        print(f"real-width chunk {ci} ({n} tokens)", flush=True)
        before = [(c.token_pos.clone(), None if ci == 0 else c.next_positions(n)) for c in model.caches]
        hidden = model.forward_chunk(ids[:, start : start + n])
        for c in model.caches:
            c.wait_for_selection()
        torch.cuda.synchronize()
        assert hidden.shape == (B, n, cfg.n_embd) and torch.isfinite(hidden.float()).all()
        for li, cache in enumerate(model.caches):
            tp = cache.token_pos[:B]
            assert cache.input_pos == start + n
            if ci == 0:
                assert torch.equal(tp, torch.arange(L, dtype=torch.int32, device=gpu).expand(B, cfg.n_query_groups, L))
                continue
            old_tp, slots = before[li]
            if ci == 1:  # initial rule: int(0.05 * 16384) = 819
                assert torch.equal(slots, torch.arange(819, 819 + n, device=gpu).expand(B, cfg.n_query_groups, n))
            want = old_tp[:B].clone()
            want.scatter_(-1, slots, torch.arange(start, start + n, dtype=torch.int32, device=gpu).expand(B, cfg.n_query_groups, n).contiguous())
            assert torch.equal(tp, want), f"layer {li} chunk {ci}: slot bookkeeping"
            assert all(len(torch.unique(tp[0, h])) == L for h in range(cfg.n_query_groups))
            s = w_sums[li][-1]
            torch.testing.assert_close(s, torch.full_like(s, float(n)), rtol=5e-4, atol=0)
            assert (cache.scores >= 0).all()
        start += n
    assert all(len(x) == 3 for x in w_sums)


def test_256_decode_steps_at_8_x_131072_slots(kvx, gpu):
    """Configuration 4 through the cache object, 256 single-token steps over B8 x 8 heads x 131072 slots
    of bf16 K/V (4.3 GB; the state is set up directly, a prefill of that length is not part of the
    configuration). Every step: the token goes to the slot chosen by the step before, the scores grow
    by weights that add up to one per row, the next slot is the row's minimum. The last step's last
    (batch, head) pair is compared with the oracle on the cache contents."""
    B, Hq, Hkv, L, D, steps = 8, 32, 8, 131072, 128, 256
    G = Hq // Hkv
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=1, device=gpu)
    torch.manual_seed(3)
    cache.k.copy_(torch.randn(B, Hkv, L, D, device=gpu, dtype=torch.bfloat16))
    cache.v.copy_(torch.randn(B, Hkv, L, D, device=gpu, dtype=torch.bfloat16))
    cache.token_pos.copy_(torch.arange(L, dtype=torch.int32, device=gpu).expand(B, Hkv, L))
    cache.batch_size, cache.current_length, cache.prefill_length = B, L, L
    cache._input_pos, cache._use_initial_rule = L, False
    cache.set_next_positions(torch.zeros((B, Hkv, 1), dtype=torch.int32, device=gpu))  # step 0 writes slot 0
    ones = torch.ones(B, Hkv, device=gpu)
    q = k = v = None
    for t in range(steps):
        if t % 64 == 0:
            print(f"decode step {t}", flush=True)
        q = torch.randn(B, Hq, 1, D, device=gpu, dtype=torch.bfloat16)
        k = torch.randn(B, Hkv, 1, D, device=gpu, dtype=torch.bfloat16)
        v = torch.randn(B, Hkv, 1, D, device=gpu, dtype=torch.bfloat16)
        slot = cache.next_positions(1)
        before = cache.scores.clone()
        before.scatter_(-1, slot, 0.0)
        out = cache.forward(q, k, v)
        grown = cache.scores - before
        assert (grown >= 0).all(), t
        torch.testing.assert_close(grown.sum(-1), ones, rtol=1e-4, atol=0)
        assert torch.equal(cache.token_pos.gather(-1, slot).squeeze(-1), torch.full((B, Hkv), L + t, dtype=torch.int32, device=gpu))
        assert torch.equal(cache.k.gather(2, slot.unsqueeze(-1).expand(-1, -1, -1, D)), k)
        nxt = cache.next_positions(1)
        assert torch.equal(cache.scores.gather(-1, nxt).squeeze(-1), cache.scores.min(-1).values), t
        assert out.shape == (B, 1, Hq * D)
    assert cache.input_pos == L + steps
    b, h = B - 1, Hkv - 1
    o_ref, w_ref = O.sdpa_in_blocks(q[b : b + 1, G * h : G * h + G].cpu(), cache.k[b : b + 1, h : h + 1].cpu(), cache.v[b : b + 1, h : h + 1].cpu(),
                                    1.0 / math.sqrt(D), L + steps - 1, None)
    got = out.view(B, Hq, D)[b, G * h : G * h + G].float().cpu()
    assert rel_err(got, o_ref[0, :, 0].float()) < 2e-2
    torch.testing.assert_close(grown[b : b + 1, h : h + 1].cpu(), w_ref, rtol=2e-3, atol=1e-9)


def _garbage_workspaces():
    for buf in _lib._workspaces.values():
        buf.fill_(0xA5)


def test_results_are_bit_reproducible(kvx, gpu):
    """No kernel uses floating-point atomics or depends on what its scratch held before: chunked prefill +
    score-sums (bf16 and 8-bit store, scattered slots, several KV splits), decode with weights, and the
    selection give identical bits on a second run over a scratch filled with garbage."""
    B, Hq, Hkv, q_len, T, D = 1, 32, 8, 1024, 32768, 128
    gen = torch.Generator().manual_seed(1)
    q = torch.randn(B, Hq, q_len, D, generator=gen).to(torch.bfloat16).to(gpu)
    k = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16).to(gpu)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16).to(gpu)
    input_pos, scale = T - q_len, 1.0 / math.sqrt(D)
    tp = scattered_positions(gen, B, Hkv, T, input_pos, q_len).to(gpu)
    kc, ks, kz = _quantize_store(kvx, gpu, k, 8)
    vc, vs, vz = _quantize_store(kvx, gpu, v, 8)
    quant = ops.QuantState(ks, kz, vs, vz)
    runs = []
    for rep in range(2):
        _garbage_workspaces()
        r = []
        r += ops.prefill_core(q, k, v, scale, input_pos, tp, return_weights=True, return_lse=True)
        r += ops.prefill_core(q, kc, vc, scale, input_pos, tp, return_weights=True, return_lse=True, quant=quant)
        r += ops.decode_core(q[:, :, :1], k, v, scale, return_weights=True, return_lse=True)
        r += ops.decode_core(q[:, :, :1], kc, vc, scale, return_weights=True, return_lse=True, quant=quant)
        torch.cuda.synchronize()
        runs.append(r)
    for i, (a, b) in enumerate(zip(*runs)):
        assert torch.equal(a, b), f"result {i} differs between two runs"
    # selection: scores += w, k smallest; and the single-slot form with its atomic minimum on integers
    scores = torch.rand(B, Hkv, T, generator=torch.Generator().manual_seed(9)).to(gpu)
    w = runs[0][1]
    for kk in (1024, 1):
        outs = []
        for rep in range(2):
            sc = scores.clone()
            nxt = torch.empty((B, Hkv, kk), dtype=torch.int32, device=gpu)
            a = _lib.H2OArgs()
            a.B, a.Hkv, a.kv_len, a.limit, a.k = B, Hkv, T, T, kk
            a.scores, a.sc_stride_b, a.sc_stride_h = sc.data_ptr(), sc.stride(0), sc.stride(1)
            a.w, a.next_index = w.data_ptr(), nxt.data_ptr()
            ws = torch.full((max(kvx.kvx_h2o_workspace_bytes(ctypes.byref(a)), 16),), 0x5A if rep else 0xFF, dtype=torch.uint8, device=gpu)
            a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
            _lib.check(kvx.kvx_h2o_update_select(ctypes.byref(a), _lib.stream_ptr(gpu)))
            torch.cuda.synchronize()
            outs.append((sc, nxt))
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
