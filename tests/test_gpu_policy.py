"""GPU parity of the eviction-policy variants (grace period ring, normalised scores, V-norm weighted
increments, Q-Hitter combination) against the CPU oracle, through the C ABI."""
import ctypes

import pytest
import torch

from helpers import rel_err
from keys_values_amd import _lib
from keys_values_amd.kvcache.h2o import (H2OKVCache, KVCacheParams, QuantizedH2OKVCache, QuantizedVLengthH2OKVCache,
                                          VLengthH2OKVCache, create_kv_cache)
from oracle import kvx_oracle as O
from oracle import policy_oracle as P

pytestmark = pytest.mark.gpu


def _sets_equal_away_from_ties(n_gpu, n_ref, compared, k):
    """Selected sets must agree unless the cut falls between values that differ in the last bits
    (the GPU's and the oracle's scores are sums in different orders)."""
    for b in range(n_ref.shape[0]):
        for h in range(n_ref.shape[1]):
            a, r = set(n_gpu[b, h, :k].tolist()), set(n_ref[b, h, :k].tolist())
            if a != r:
                srt = torch.sort(compared[b, h]).values
                cut = srt[k - 1].item()
                tol = 2e-3 * max(abs(cut), 1e-6)
                assert all(abs(compared[b, h, i].item() - cut) < tol for i in a ^ r), \
                    f"selection differs away from a tie at ({b},{h}): {sorted(a ^ r)}"


def _store(cache):
    """What the cache holds, as bf16 rows."""
    if not cache.quantized:
        return cache.k.cpu(), cache.v.cpu()
    unpack = O.uncompress4 if cache.num_bits == 4 else (lambda c: c)
    return (O.dequantize_rows(unpack(cache.k.cpu()), cache.k_scale.cpu(), cache.k_zp.cpu()),
            O.dequantize_rows(unpack(cache.v.cpu()), cache.v_scale.cpu(), cache.v_zp.cpu()))


def _run_steps(gpu, cache, ref, q, k, v, n_prefill, steps):
    B, Hq, D = q.shape[0], q.shape[1], q.shape[3]
    ref.prefill(q[:, :, :n_prefill], k[:, :, :n_prefill], v[:, :, :n_prefill])
    cache.forward(q[:, :, :n_prefill].to(gpu), k[:, :, :n_prefill].to(gpu), v[:, :, :n_prefill].to(gpu))
    pos = n_prefill
    for num in steps:
        assert cache.max_forward_length() == ref.max_forward_length()
        if callable(num):  # a step size drawn from what the cache accepts now
            num = num(ref.max_forward_length())
        sl = slice(pos, pos + num)
        had_choice = ref.next_index is not None
        o_ref, w_ref, index = ref.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        if had_choice:
            # evict the oracle's slots so that both caches stay comparable (the GPU's own choice was checked below)
            cache.set_next_positions(index)
        o = cache.forward(q[:, :, sl].to(gpu), k[:, :, sl].to(gpu), v[:, :, sl].to(gpu))
        torch.cuda.synchronize()
        assert cache.input_pos == ref.input_pos and cache.current_length == ref.current_length
        assert cache.next_grace_pos == ref.next_grace_pos
        assert torch.equal(cache.token_pos.cpu(), ref.token_pos), f"token positions differ after a step of {num}"
        kk, vv = _store(cache)
        assert torch.equal(kk, ref.k) and torch.equal(vv, ref.v), f"stored rows differ after a step of {num}"
        assert rel_err(o.float().cpu().view(B, num, Hq, D).transpose(1, 2), o_ref.float()) < 2e-2
        torch.testing.assert_close(cache.scores.cpu(), ref.scores, rtol=2e-3, atol=1e-5)
        if cache.v_norm is not None:
            torch.testing.assert_close(cache.v_norm.cpu(), ref.buffers["v_norm"], rtol=1e-5, atol=1e-6)
        if cache.q_errors is not None:
            torch.testing.assert_close(cache.q_errors.cpu(), ref.buffers["q_errors"], rtol=1e-5, atol=1e-6)
        if ref.next_index is not None:
            # the cache chooses as many slots as the step after may need at once (one after a single token)
            # and selects again when asked for more; the oracle keeps the reference's whole list
            assert cache._select_k == ref.next_index.shape[-1]
            kk_sel = cache._next_count
            assert 1 <= kk_sel <= cache._select_k
            got = cache._next_index[:B, :, :kk_sel].cpu().long()
            assert int(got.max()) < cache.cache_length - cache.grace_period, "a ring slot was chosen for eviction"
            _sets_equal_away_from_ties(got, ref.next_index, ref.compared, kk_sel)
        pos += num


def _inputs(seed, B, Hq, Hkv, total, D, spread=False):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, total, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(B, Hkv, total, D, generator=gen)
    v = torch.randn(B, Hkv, total, D, generator=gen)
    if spread:  # rows of different size: spreads the V norms and the quantisation errors
        k = k * (0.5 + 3 * torch.rand(B, Hkv, total, 1, generator=gen))
        v = v * (0.5 + 3 * torch.rand(B, Hkv, total, 1, generator=gen))
    return q, k.to(torch.bfloat16), v.to(torch.bfloat16)


@pytest.mark.parametrize("quantized", [False, True])
def test_grace_period_steps(gpu, quantized):
    """test/kvcache/test_h2o.py:49-106 shapes of behaviour at kernel-sized heads: a cache that fills
    up after the prefill, then steps shorter than, equal to and longer than the grace period."""
    B, Hq, Hkv, L, D, gp, chunk = 2, 8, 2, 512, 64, 24, 64
    steps = (40, 1, 1, 7, 24, 64, 30, 1, 17, 64, 3, 1)
    q, k, v = _inputs(7, B, Hq, Hkv, L + sum(steps), D)
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=chunk, grace_period=gp, quantized=quantized, device=gpu)
    ref = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, grace_period=gp, quantized=quantized)
    _run_steps(gpu, cache, ref, q, k, v, L - 40, steps)
    # the invariants the reference's own test asserts
    tp = cache.token_positions().cpu()
    last = cache.input_pos - 1
    assert sorted(tp[0, 0, L - gp:].tolist()) == list(range(last - gp + 1, last + 1))
    assert int(tp[:, :, : L - gp].max()) <= last - gp


@pytest.mark.parametrize("name,kwargs", [
    ("h2o-vlen-default", dict()),
    ("h2o-vlen-torch-quantized8", dict(grace_period=9, normalize_scores=True)),
    ("qh2o-torch-quantized8", dict(combination_constant=0.3)),
    ("qh2o-vlen-torch-quantized8", dict(grace_period=16, normalize_scores=True)),
    ("h2o-torch-quantized4", dict()),
    ("qh2o-vlen-torch-quantized4", dict(grace_period=16)),
])
def test_policy_variants_chunked_steps(gpu, name, kwargs):
    B, Hq, Hkv, L, D, chunk = 2, 8, 2, 384, 128, 32
    steps = (32, 5, 32, 1, 20, 32, 1, 1, 32)
    q, k, v = _inputs(len(name), B, Hq, Hkv, L + sum(steps), D, spread=True)
    cache = create_kv_cache(name, KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=chunk, device=gpu, **kwargs)
    ref = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, quantized=cache.quantized, v_length=cache.v_length,
                              q_hitter=cache.q_hitter, combination_constant=cache.combination_constant,
                              grace_period=cache.grace_period, normalize_scores=cache.normalize_scores,
                              num_bits=cache.num_bits or 8)
    _run_steps(gpu, cache, ref, q, k, v, L, steps)


def _random_policies(n, seed):
    import random

    rnd = random.Random(seed)
    cases = []
    for i in range(n):
        Hkv = rnd.choice([1, 2, 3])
        L = rnd.choice([130, 256, 333, 600])
        chunk = rnd.choice([1, 8, 33, 64])
        quantized = rnd.random() < 0.5
        cases.append(dict(i=i, B=rnd.choice([1, 2]), Hq=Hkv * rnd.choice([1, 2, 4]), Hkv=Hkv, L=L, D=rnd.choice([64, 128]), chunk=chunk,
                          gp=rnd.choice([0, 0, 3, chunk, 40]), quantized=quantized, bits=rnd.choice([4, 8]) if quantized else 8,
                          v_length=rnd.random() < 0.4, q_hitter=quantized and rnd.random() < 0.5, normalize=rnd.random() < 0.4,
                          c=rnd.choice([0.25, 0.5, 0.8]), short=rnd.randint(0, 50)))
    return cases


@pytest.mark.parametrize("cfg", _random_policies(16, 424242), ids=lambda c: "-".join(f"{k}{v}" for k, v in c.items()))
def test_random_policy_configurations(gpu, cfg):
    """Seeded mixes of the options the fixed cases vary one at a time, with step sizes drawn from what
    the cache accepts at each step (test/kvcache/test_h2o.py:49-106, test/kvcache/test_attn_weights.py)."""
    import random

    rnd = random.Random(cfg["i"])
    B, Hq, Hkv, L, D, chunk = cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["L"], cfg["D"], cfg["chunk"]
    nsteps = 14
    steps = [lambda m: rnd.randint(1, min(m, chunk))] * nsteps
    q, k, v = _inputs(900 + cfg["i"], B, Hq, Hkv, L + nsteps * chunk, D, spread=True)
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=chunk, normalize_scores=cfg["normalize"], grace_period=cfg["gp"],
                       quantized=cfg["quantized"], num_bits=cfg["bits"], v_length=cfg["v_length"], q_hitter=cfg["q_hitter"],
                       combination_constant=cfg["c"], device=gpu)
    ref = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, quantized=cfg["quantized"], v_length=cfg["v_length"],
                              q_hitter=cfg["q_hitter"], combination_constant=cfg["c"], grace_period=cfg["gp"],
                              normalize_scores=cfg["normalize"], num_bits=cfg["bits"])
    _run_steps(gpu, cache, ref, q, k, v, L - cfg["short"], steps)


@pytest.mark.parametrize("cls,kwargs", [
    (VLengthH2OKVCache, dict()),
    (QuantizedH2OKVCache, dict(grace_period=5)),
    (QuantizedVLengthH2OKVCache, dict(normalize_scores=True)),
    (H2OKVCache, dict(grace_period=7)),
    (H2OKVCache, dict(quantized=True, num_bits=4, grace_period=3)),
])
def test_policy_variants_single_token_steps(gpu, cls, kwargs):
    # max_chunk_size = 1: the argmin form of the selection (and, for plain H2O, the fused decode step)
    B, Hq, Hkv, L, D = 2, 8, 4, 300, 128
    steps = (1,) * 12
    q, k, v = _inputs(3, B, Hq, Hkv, L + len(steps), D, spread=True)
    cache = cls(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=1, device=gpu, **kwargs)
    ref = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=1, quantized=cache.quantized, v_length=cache.v_length,
                              q_hitter=cache.q_hitter, combination_constant=cache.combination_constant,
                              grace_period=cache.grace_period, normalize_scores=cache.normalize_scores,
                              num_bits=cache.num_bits or 8)
    _run_steps(gpu, cache, ref, q, k, v, L, steps)


def _gpu_update(kvx, gpu, scores, w, limit, k, v_norm=None, q_errors=None, combination=0.5, q_len=1, normalize=False,
                token_pos=None, input_pos=0, prefill_len=0):
    B, Hkv, L = scores.shape
    kv_len = w.shape[-1]
    dev = lambda t: None if t is None else t.contiguous().to(gpu)  # noqa: E731
    sc_g, w_g, vn_g, qe_g = dev(scores), dev(w), dev(v_norm), dev(q_errors)
    tp_g = None if token_pos is None else token_pos.to(torch.int32).to(gpu)
    nxt = torch.empty((B, Hkv, k), dtype=torch.int32, device=gpu)
    a = _lib.H2OArgs()
    a.B, a.Hkv, a.kv_len, a.limit, a.k = B, Hkv, kv_len, limit, k
    a.normalize, a.input_pos, a.prefill_len = int(normalize), input_pos, prefill_len
    a.scores, a.sc_stride_b, a.sc_stride_h = sc_g.data_ptr(), sc_g.stride(0), sc_g.stride(1)
    a.w = w_g.data_ptr()
    if tp_g is not None:
        a.token_pos, a.tp_stride_b, a.tp_stride_h = tp_g.data_ptr(), tp_g.stride(0), tp_g.stride(1)
    a.v_norm, a.q_errors, a.q_len, a.combination = _lib.ptr(vn_g), _lib.ptr(qe_g), q_len, combination
    a.next_index = nxt.data_ptr()
    nb = kvx.kvx_h2o_workspace_bytes(ctypes.byref(a))
    ws = torch.empty(max(nb, 16), dtype=torch.uint8, device=gpu)
    a.workspace, a.workspace_bytes = ws.data_ptr(), nb
    _lib.check(kvx.kvx_h2o_update_select(ctypes.byref(a), _lib.stream_ptr(gpu)))
    torch.cuda.synchronize()
    return sc_g.cpu(), nxt.cpu().long()


@pytest.mark.parametrize("B,Hkv,L,limit,k,vlen,qh,normalize", [
    (2, 4, 5000, 4900, 1, True, False, False),
    (2, 4, 5000, 5000, 256, True, True, True),
    (1, 8, 32768, 32768 - 64, 1024, False, True, False),
    (3, 2, 777, 700, 1, True, True, True),
    (1, 2, 50000, 50000, 128, True, True, False),   # rows too long for the LDS-resident keys
])
def test_update_select_variants_direct(kvx, gpu, B, Hkv, L, limit, k, vlen, qh, normalize):
    gen = torch.Generator().manual_seed(L + k)
    scores = torch.rand(B, Hkv, L, generator=gen) * 3
    w = torch.rand(B, Hkv, L, generator=gen) ** 4
    vn = (torch.rand(B, Hkv, L, generator=gen) * 5 + 0.1) if vlen else None
    qe = (torch.rand(B, Hkv, L, generator=gen) * 0.2) if qh else None
    tp = torch.stack([torch.randperm(3 * L, generator=gen)[:L] for _ in range(B * Hkv)]).view(B, Hkv, L).to(torch.int32)
    input_pos, prefill_len, q_len, c = 3 * L + 9, L // 3, 17, 0.4
    s_ref = scores.clone()
    n_ref, compared = P.update_select(s_ref, w, L, limit, k, normalize=normalize, token_pos=tp, input_pos=input_pos,
                                      prefill_len=prefill_len, v_norm=vn, q_errors=qe, combination=c, q_len=q_len)
    s_gpu, n_gpu = _gpu_update(kvx, gpu, scores, w, limit, k, vn, qe, c, q_len, normalize, tp, input_pos, prefill_len)
    torch.testing.assert_close(s_gpu, s_ref, rtol=1e-5, atol=1e-7)
    if vlen:  # the increments of a row sum to the number of queries
        torch.testing.assert_close((s_gpu - scores).sum(-1), torch.full((B, Hkv), float(q_len)), rtol=1e-4, atol=1e-4)
    else:
        assert torch.equal(s_gpu, s_ref)
    _sets_equal_away_from_ties(n_gpu, n_ref, compared, k)
    # ascending order of the compared values among the chosen slots
    chosen = compared.gather(-1, n_gpu)
    assert bool((chosen[..., 1:] >= chosen[..., :-1] - 2e-3 * chosen.abs().max()).all())


def test_q_hitter_extremes_direct(kvx, gpu):
    # c = 1 is plain H2O; c = 0 evicts the largest quantisation errors (both exact: no sums involved)
    gen = torch.Generator().manual_seed(8)
    B, Hkv, L, k = 2, 3, 2000, 100
    scores = torch.rand(B, Hkv, L, generator=gen)
    w = torch.zeros(B, Hkv, L)
    qe = torch.rand(B, Hkv, L, generator=gen)
    _, n1 = _gpu_update(kvx, gpu, scores, w, L, k, None, qe, 1.0)
    _, n0 = _gpu_update(kvx, gpu, scores, w, L, k, None, qe, 0.0)
    for b in range(B):
        for h in range(Hkv):
            assert set(n1[b, h].tolist()) == set(torch.argsort(scores[b, h], stable=True)[:k].tolist())
            assert set(n0[b, h].tolist()) == set(torch.argsort(qe[b, h], descending=True, stable=True)[:k].tolist())


def test_cache_write_ring_rejects_bad_arguments(kvx, gpu):
    a = _lib.CacheWriteArgs()
    a.B, a.Hkv, a.num, a.D, a.cache_len, a.input_pos = 1, 1, 4, 64, 32, 40
    buf = torch.zeros(32 * 64, dtype=torch.bfloat16, device=gpu)
    idx = torch.zeros(4, dtype=torch.int32, device=gpu)
    for f in ("index", "token_pos"):
        setattr(a, f, idx.data_ptr())
    for f in ("key", "value", "k_cache", "v_cache"):
        setattr(a, f, buf.data_ptr())
    a.key_stride_t = a.value_stride_t = a.kc_stride_t = a.vc_stride_t = 64
    a.grace_num, a.grace_period = 5, 8  # more ring slots than new tokens
    assert kvx.kvx_cache_write(ctypes.byref(a), None) == _lib.KVX_ERR_INVALID
    a.grace_num = 2  # ring move without the ring slots
    assert kvx.kvx_cache_write(ctypes.byref(a), None) == _lib.KVX_ERR_INVALID and b"grace_slots" in kvx.kvx_last_error()
    a.grace_num, a.q_errors = 0, buf.data_ptr()  # quantisation errors of a bf16 store
    assert kvx.kvx_cache_write(ctypes.byref(a), None) == _lib.KVX_ERR_INVALID


def test_factory_names_and_errors(gpu):
    params = KVCacheParams(1, 2, 64, 64, 4)
    assert isinstance(create_kv_cache("h2o-default", params, device=gpu), H2OKVCache)
    c = create_kv_cache("qh2o-vlen-torch-quantized8", params, device=gpu, grace_period=3)
    assert c.quantized and c.v_length and c.q_hitter and c.grace_period == 3 and c.max_forward_length is not None
    with pytest.raises(TypeError):
        create_kv_cache("qh2o-default", params, device=gpu)  # keys_values/kvcache/qh2o.py:95-96
    with pytest.raises(NotImplementedError):
        create_kv_cache("lastrec-default", params, device=gpu)
    with pytest.raises(NotImplementedError):
        create_kv_cache("h2o-bnb-quantized4", params, device=gpu)
    with pytest.raises(ValueError):
        H2OKVCache(params, grace_period=64, device=gpu)
    with pytest.raises(ValueError):
        QuantizedH2OKVCache(params, combination_constant=1.5, device=gpu)


@pytest.mark.parametrize("kwargs", [dict(), dict(grace_period=6, quantized=True)])
def test_replay_log(gpu, kwargs):
    """test/kvcache/test_h2o.py:227-343: the log holds the token chunks and, for every position from
    cache_length on, the slot its K/V went to; blocks of `replay_log_blocksize` positions."""
    B, Hq, Hkv, L, D, chunk, bs = 2, 8, 2, 128, 64, 16, 10
    steps = (5, 16, 1, 1, 16, 7, 16, 1, 3)
    q, k, v = _inputs(11, B, Hq, Hkv, L + sum(steps), D)
    gen = torch.Generator().manual_seed(1)
    tokens = torch.randint(0, 128, (B, L + sum(steps)), generator=gen)
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=chunk, replay_log_blocksize=bs, device=gpu, **kwargs)
    ref = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, replay_log_blocksize=bs,
                              grace_period=cache.grace_period, quantized=cache.quantized)
    assert cache.get_replay_log() is None and not cache.do_replay_logging
    cache.switch_replay_logging(True)
    n0 = L - 5
    with pytest.raises(ValueError):  # logging needs the token indices
        cache.forward(q[:, :, :n0].to(gpu), k[:, :, :n0].to(gpu), v[:, :, :n0].to(gpu))
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=chunk, replay_log_blocksize=bs, device=gpu, **kwargs)
    cache.switch_replay_logging(True)
    ref.prefill(q[:, :, :n0], k[:, :, :n0], v[:, :, :n0])
    cache.forward(q[:, :, :n0].to(gpu), k[:, :, :n0].to(gpu), v[:, :, :n0].to(gpu), tokens[:, :n0].to(gpu))
    log = cache.get_replay_log()
    assert len(log) == n0 and log.slot_positions == [] and log.cache_length == L and log.grace_period == cache.grace_period
    pos, used = n0, []
    for num in steps:
        sl = slice(pos, pos + num)
        had_choice = ref.next_index is not None
        _, _, index = ref.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        if had_choice:
            cache.set_next_positions(index)
        cache.forward(q[:, :, sl].to(gpu), k[:, :, sl].to(gpu), v[:, :, sl].to(gpu), tokens[:, sl].to(gpu))
        if pos >= L:
            used.append(index)
        pos += num
        log = cache.get_replay_log()
        assert len(log) == pos == cache.input_pos
        want = ref.replay_log.finalize(pos)
        assert len(log.slot_positions) == len(want)
        for got, w in zip(log.slot_positions, want):
            assert got.dtype == torch.uint32 and tuple(got.shape) == tuple(w.shape)
            assert torch.equal(got.view(torch.int32).cpu().long(), w)
    flat = torch.cat(used, dim=-1)
    assert torch.equal(torch.cat([b.view(torch.int32).cpu().long() for b in log.slot_positions], dim=-1), flat)
    assert torch.equal(log.extract_index(L + 3, 25).cpu(), flat[:, :, 3:28])
    assert log.extract_index(L, 1, dtype=torch.int32).dtype == torch.int32
    for c, (a, b) in zip(log.token_chunks, [(0, n0)] + [(n0 + sum(steps[:i]), n0 + sum(steps[: i + 1])) for i in range(len(steps))]):
        assert torch.equal(c.cpu(), tokens[:, a:b])
    with pytest.raises(ValueError):
        log.extract_index(L - 1, 1)
    with pytest.raises(ValueError):
        log.extract_index(pos - 1, 5)
    # switching on in the middle of a run needs a new prefill (keys_values/kvcache/attn_weights.py:623-628)
    cache.switch_replay_logging(False)
    assert cache.get_replay_log() is None
    cache.switch_replay_logging(True)
    with pytest.raises(IndexError):
        cache.forward(q[:, :, :1].to(gpu), k[:, :, :1].to(gpu), v[:, :, :1].to(gpu), tokens[:, :1].to(gpu))
    with pytest.raises(ValueError):
        H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), replay_log_blocksize=0, device=gpu)
