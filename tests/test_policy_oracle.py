"""Pins of the policy-variant oracle (oracle/policy_oracle.py) on the CPU: an independent per-slot
model for the grace period, closed forms and brute force for the V-norm weighting and the Q-Hitter
combination. None of these retype the oracle's own expressions."""
import math

import numpy as np
import pytest
import torch

from oracle import kvx_oracle as O
from oracle import policy_oracle as P


def _inputs(seed, B, Hq, Hkv, total, D):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, total, D, generator=gen).to(torch.bfloat16)
    k = torch.randn(B, Hkv, total, D, generator=gen).to(torch.bfloat16)
    v = torch.randn(B, Hkv, total, D, generator=gen).to(torch.bfloat16)
    return q, k, v


def test_no_grace_no_variant_is_the_h2o_oracle():
    B, Hq, Hkv, L, D, chunk = 2, 4, 2, 64, 16, 8
    q, k, v = _inputs(0, B, Hq, Hkv, L + 5 * chunk, D)
    a = O.H2OCacheOracle(B, Hq, Hkv, L, D, dtype=torch.bfloat16, max_chunk_size=chunk)
    b = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk)
    n0 = L - 3  # the cache fills up during the first step after the prefill
    oa = a.prefill(q[:, :, :n0], k[:, :, :n0], v[:, :, :n0])
    ob = b.prefill(q[:, :, :n0], k[:, :, :n0], v[:, :, :n0])
    assert torch.equal(oa, ob)
    pos = n0
    for num in (3, chunk, 1, chunk, 5):
        sl = slice(pos, pos + num)
        ra = a.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        rb = b.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        for x, y in zip(ra, rb):
            assert torch.equal(x, y)
        assert torch.equal(a.token_pos, b.token_pos) and torch.equal(a.scores, b.scores)
        assert torch.equal(a.k, b.k) and torch.equal(a.v, b.v)
        assert torch.equal(a.next_index, b.next_index)
        pos += num


@pytest.mark.parametrize("gp,steps", [(5, (1, 1, 3, 5, 7, 2, 8, 1, 4, 6, 5, 1)), (1, (1, 2, 1, 4, 1)), (13, (1,) * 40)])
def test_grace_period_against_a_per_slot_model(gp, steps):
    """The model keeps, per (b, h), a dict token -> (key row, value row, score) and a list of the
    last `gp` tokens; it never computes a slot index. After every step the oracle's buffers, read
    back through its token positions, must hold exactly the model's content, the ring must hold the
    most recent tokens oldest-first from next_grace_pos, and the invariants of
    test/kvcache/test_h2o.py:87-106 must hold."""
    B, Hq, Hkv, L, D = 2, 4, 2, 48, 8
    total = L + sum(steps)
    q, k, v = _inputs(gp, B, Hq, Hkv, total, D)
    ora = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=8, grace_period=gp)
    ora.prefill(q[:, :, :L], k[:, :, :L], v[:, :, :L])
    model = [[{t: [k[b, h, t], v[b, h, t], 0.0] for t in range(L)} for h in range(Hkv)] for b in range(B)]
    pos = L
    for num in steps:
        sl = slice(pos, pos + num)
        before_tp = ora.token_pos.clone()
        _, w, index = ora.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        assert int(index.max()) < L - gp, "evicted slots must lie outside the ring"
        for b in range(B):
            for h in range(Hkv):
                m = model[b][h]
                for t in before_tp[b, h, index[b, h]].tolist():  # tokens in the evicted slots
                    del m[t]
                for t in range(pos, pos + num):
                    m[t] = [k[b, h, t], v[b, h, t], 0.0]
                tp = ora.token_pos[b, h].tolist()
                assert sorted(tp) == sorted(m.keys()), "token set differs"
                for slot, t in enumerate(tp):
                    m[t][2] += float(w[b, h, slot])
                    assert torch.equal(ora.k[b, h, slot], m[t][0]) and torch.equal(ora.v[b, h, slot], m[t][1])
                    assert abs(float(ora.scores[b, h, slot]) - m[t][2]) <= 1e-5 * max(1.0, abs(m[t][2]))
                # the ring: last gp tokens, oldest first from next_grace_pos
                prefix = L - gp
                start = ora.next_grace_pos - prefix
                ring = [tp[prefix + (start + i) % gp] for i in range(gp)]
                last = pos + num - 1
                assert ring == list(range(last - gp + 1, last + 1))
                assert all(0 <= x <= last - gp for x in tp[:prefix])
        pos += num


@pytest.mark.parametrize("bits", [8, 4])
def test_quantised_ring_row_is_written_like_a_new_row(bits):
    """A row that leaves the ring is read as bf16 values and written by the same write as the new rows
    (keys_values/kvcache/attn_weights.py:578-590, keys_values/kvcache/quant_buffers.py:732-775): its
    second stay in the store holds quantise(dequantise(.)) of the first, once; rows that are not
    written keep their content."""
    B, Hq, Hkv, L, D, gp = 1, 2, 1, 32, 16, 4
    q, k, v = _inputs(11, B, Hq, Hkv, L + 12, D)
    ora = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=4, grace_period=gp, quantized=True, num_bits=bits)
    ora.prefill(q[:, :, :L], k[:, :, :L], v[:, :, :L])
    first = {t: O.dequantize_rows(*O.quantize_rows(k[0, 0, t : t + 1], bits))[0] for t in range(L + 12)}
    second = {t: O.dequantize_rows(*O.quantize_rows(first[t].unsqueeze(0), bits))[0] for t in first}
    moved = set()
    changed = 0
    pos = L
    for num in (3, 4, 1, 4):
        ora.forward(q[:, :, pos : pos + num], k[:, :, pos : pos + num], v[:, :, pos : pos + num])
        pos += num
        moved |= {t for t in range(L - gp, pos - gp)}  # tokens that have left the ring by now
        for slot, t in enumerate(ora.token_pos[0, 0].tolist()):
            want = second[t] if t in moved else first[t]
            assert torch.equal(ora.k[0, 0, slot], want), (t, slot)
            changed += int(t in moved and not torch.equal(first[t], second[t]))
    assert changed > 0, "the case must contain a row for which writing twice is not the identity"


def test_v_length_with_equal_norms_is_plain_h2o():
    # sum_k W = q_len, so a constant |v| cancels: instantaneous score == W
    B, Hq, Hkv, L, D, chunk = 1, 4, 2, 64, 16, 8
    q, k, v = _inputs(5, B, Hq, Hkv, L + 4 * chunk, D)
    v = (v.float() / torch.linalg.vector_norm(v.float(), dim=-1, keepdim=True)).to(torch.bfloat16)
    plain = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk)
    vlen = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, v_length=True)
    plain.prefill(q[:, :, :L], k[:, :, :L], v[:, :, :L])
    vlen.prefill(q[:, :, :L], k[:, :, :L], v[:, :, :L])
    pos = L
    for _ in range(4):
        sl = slice(pos, pos + chunk)
        if vlen.next_index is not None:
            vlen.next_index = plain.next_index  # same evictions, so that the score buffers stay comparable
        _, _, idx = plain.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        before = vlen.scores.clone()
        before.scatter_(-1, idx, 0.0)
        vlen.forward(q[:, :, sl], k[:, :, sl], v[:, :, sl])
        # bf16 rounding leaves the norms equal to within 2^-8
        torch.testing.assert_close(vlen.scores, plain.scores, rtol=2e-2, atol=1e-4)
        torch.testing.assert_close((vlen.scores - before).sum(-1), torch.full((B, Hkv), float(chunk)), rtol=1e-5, atol=1e-5)
        pos += chunk


def test_v_length_scores_by_brute_force():
    # test/kvcache/test_h2o.py:109-225: no eviction, every token's score recomputed from full
    # attention over the tokens so far, in float64 loops
    B, Hq, Hkv, L, D, n0, total = 1, 4, 2, 40, 8, 20, 36
    q, k, v = _inputs(9, B, Hq, Hkv, total, D)
    ora = P.PolicyCacheOracle(B, Hq, Hkv, L, D, v_length=True)
    ora.prefill(q[:, :, :n0], k[:, :, :n0], v[:, :, :n0])
    expect = np.zeros((B, Hkv, total))
    vn = np.sqrt((v.double().numpy() ** 2).sum(-1))
    for pos in range(n0, total):
        ora.forward(q[:, :, pos : pos + 1], k[:, :, pos : pos + 1], v[:, :, pos : pos + 1])
        _, W, _ = O.weights_bruteforce_f64(q[:, :, pos : pos + 1], k[:, :, : pos + 1], v[:, :, : pos + 1], 1 / math.sqrt(D), pos, None)
        s = W * vn[:, :, : pos + 1]
        expect[:, :, : pos + 1] += s / s.sum(-1, keepdims=True)
    np.testing.assert_allclose(ora.scores[:, :, :total].double().numpy(), expect, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(ora.buffers["v_norm"][:, :, :total].double().numpy(), vn, rtol=1e-6)


def _bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest-even bfloat16, as float32 (bit arithmetic, no torch)."""
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def test_quantization_error_by_loops():
    gen = torch.Generator().manual_seed(11)
    x = (torch.randn(6, 64, generator=gen) * 3).to(torch.bfloat16)
    got = O.quantization_error(x).numpy()
    xs = x.float().numpy()
    for r in range(xs.shape[0]):
        row = xs[r]
        mn, mx = np.float32(row.min()), np.float32(row.max())
        scale = max(np.float32((mx - mn) / np.float32(255.0)), np.float32(1.1920929e-07))
        zp = -int(np.rint(np.float32(mn / scale)))
        acc = 0.0
        for d in range(row.size):
            code = min(max(int(np.rint(np.float32(row[d] * np.float32(np.float32(1.0) / scale)))) + zp, 0), 255)
            dq = _bf16_round(np.array([np.float32(code - zp) * scale], dtype=np.float32))[0]
            diff = _bf16_round(np.array([row[d] - dq], dtype=np.float32))[0]
            acc += float(diff) ** 2
        assert abs(got[r] - math.sqrt(acc)) <= 1e-5 * math.sqrt(acc) + 1e-9


def _qh_pair(c, seed=21):
    B, Hq, Hkv, L, D, chunk = 2, 4, 2, 64, 16, 8
    q, k, v = _inputs(seed, B, Hq, Hkv, L + 3 * chunk, D)
    gen = torch.Generator().manual_seed(seed + 1)
    k = (k.float() * (1 + 4 * torch.rand(B, Hkv, k.shape[2], 1, generator=gen))).to(torch.bfloat16)  # spread the quantisation errors
    plain = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, quantized=True)
    qh = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, quantized=True, q_hitter=True, combination_constant=c)
    for o in (plain, qh):
        o.prefill(q[:, :, :L], k[:, :, :L], v[:, :, :L])
        o.forward(q[:, :, L : L + chunk], k[:, :, L : L + chunk], v[:, :, L : L + chunk])
    return plain, qh, chunk


def test_q_hitter_constant_one_is_plain_h2o():
    plain, qh, chunk = _qh_pair(1.0)
    assert torch.equal(qh.scores, plain.scores)
    for b in range(2):
        for h in range(2):
            assert set(qh.next_index[b, h].tolist()) == set(plain.next_index[b, h].tolist())
    assert float(qh.compared.min()) >= 0.0 and float(qh.compared.max()) <= 1.0


def test_q_hitter_constant_zero_evicts_the_largest_errors():
    _, qh, chunk = _qh_pair(0.0)
    qe = qh.buffers["q_errors"]
    for b in range(2):
        for h in range(2):
            want = set(torch.argsort(qe[b, h], descending=True, stable=True)[:chunk].tolist())
            assert set(qh.next_index[b, h].tolist()) == want
    assert float(qh.compared.min()) >= 0.5 - 1e-6 and float(qh.compared.max()) <= 1.0 + 1e-6


def test_q_hitter_values_stay_in_range_and_errors_follow_the_slots():
    _, qh, chunk = _qh_pair(0.3)
    c = 0.3
    assert float(qh.compared.min()) >= (1 - c) / 2 - 1e-6 and float(qh.compared.max()) <= 1.0 + 1e-6
    # q_errors of a slot = error of the row it holds, recomputed from the stored token position
    B, Hq, Hkv, L, D = qh.B, qh.Hq, qh.Hkv, qh.L, qh.D
    q, k, v = _inputs(21, B, Hq, Hkv, L + 3 * chunk, D)
    gen = torch.Generator().manual_seed(22)
    k = (k.float() * (1 + 4 * torch.rand(B, Hkv, k.shape[2], 1, generator=gen))).to(torch.bfloat16)
    err = O.quantization_error(k) + O.quantization_error(v)
    torch.testing.assert_close(qh.buffers["q_errors"], err.gather(-1, qh.token_pos.long()), rtol=0, atol=0)


def test_replay_log_blocks_are_the_concatenated_slots():
    gen = torch.Generator().manual_seed(4)
    L, bs = 50, 7
    log = P.ReplayLogOracle(L, bs)
    chunks = []
    pos = L
    for num in (1, 3, 7, 20, 1, 6, 2, 15):
        idx = torch.randint(0, L, (2, 3, num), generator=gen)
        log.append_position_index(idx, pos)
        chunks.append(idx)
        pos += num
    flat = torch.cat(chunks, dim=-1)
    total = flat.shape[-1]
    blocks = log.finalize(pos)
    assert all(b.shape[-1] == bs for b in blocks[:-1]) and blocks[-1].shape[-1] == total - bs * (len(blocks) - 1)
    assert torch.equal(torch.cat(blocks, dim=-1), flat)
    for start in range(total):
        for num in (1, 2, bs, bs + 1, total - start):
            if start + num <= total:
                assert torch.equal(log.extract_index(L + start, num), flat[:, :, start : start + num])
    assert log.finalize(L) == []


# ---- normalised scores (keys_values/kvcache/h2o.py:183-196) ------------------------------------------


def _normalised_choice_by_loop(score_rows, pos_rows, limit, k, input_pos_after, prefill_len, clamp_shift=1, pos_shift=0):
    """Per-slot restatement with numpy float32 scalars: a slot holding the token at position p with
    cumulative score s is compared by s / float32(input_pos_after - max(p, prefill_len - 1)); the k
    smallest (value, slot) tuples. clamp_shift / pos_shift build the off-by-one variants a mistake would
    produce, to show that the test data tells them apart."""
    out = []
    for srow, prow in zip(score_rows, pos_rows):
        cands = []
        for slot in range(limit):
            resident_since = max(int(prow[slot]), prefill_len - clamp_shift)
            den = np.float32(input_pos_after - pos_shift - resident_since)
            cands.append((np.float32(srow[slot]) / den, slot))
        cands.sort()
        out.append([slot for _, slot in cands[:k]])
    return out


def test_normalised_selection_against_a_per_slot_loop():
    """Both restatements of the normalised selection (oracle.kvx_oracle.h2o_update_select and
    oracle.policy_oracle.update_select) against explicit per-slot loops. A third of the slots hold tokens
    of the prefill (position < prefill_len - 1: the clamp decides their residency), the others later
    tokens; the case is built so that clamping at prefill_len instead of prefill_len - 1, or dividing
    by the position count before this step's advance, selects a different set."""
    B, Hkv, L, limit, k = 2, 3, 96, 90, 17
    prefill_len, q_len = 40, 4
    input_pos_after = 200
    gen = torch.Generator().manual_seed(21)
    tp = torch.empty(B, Hkv, L, dtype=torch.int32)
    for b in range(B):
        for h in range(Hkv):
            old = torch.randperm(prefill_len - 1, generator=gen)[: L // 3]              # < prefill_len - 1
            new = prefill_len - 1 + torch.randperm(input_pos_after - q_len - prefill_len, generator=gen)[: L - L // 3]  # >= prefill_len - 1
            tp[b, h] = torch.cat((old, new))[torch.randperm(L, generator=gen)].to(torch.int32)
    assert (tp < prefill_len - 1).any() and (tp >= prefill_len - 1).any() and int(tp.max()) < input_pos_after
    # scores proportional to the residency, so that all ratios are close and an off-by-one in the
    # denominator reorders them; a little noise keeps exact ties away
    res = (input_pos_after - tp.clamp_min(prefill_len - 1)).float()
    scores0 = res * (1.0 + 0.02 * torch.rand(B, Hkv, L, generator=gen))
    w = 0.01 * torch.rand(B, Hkv, L, generator=gen)
    summed = (scores0 + w)  # fp32 add, as the update does
    flat_s = summed.view(B * Hkv, L).numpy()
    flat_p = tp.view(B * Hkv, L).numpy()
    want = _normalised_choice_by_loop(flat_s, flat_p, limit, k, input_pos_after, prefill_len)
    s1 = scores0.clone()
    got1 = O.h2o_update_select(s1, w, L, limit, k, normalize=True, token_pos=tp, input_pos=input_pos_after, prefill_len=prefill_len)
    s2 = scores0.clone()
    got2, compared = P.update_select(s2, w, L, limit, k, normalize=True, token_pos=tp, input_pos=input_pos_after, prefill_len=prefill_len)
    assert torch.equal(s1, summed) and torch.equal(s2, summed)
    assert got1.view(B * Hkv, k).tolist() == want
    assert got2.view(B * Hkv, k).tolist() == want
    for r in range(B * Hkv):  # the compared values themselves, element by element
        for slot in range(limit):
            den = np.float32(input_pos_after - max(int(flat_p[r, slot]), prefill_len - 1))
            assert compared.view(B * Hkv, limit)[r, slot].item() == float(np.float32(flat_s[r, slot]) / den)
    # the plausible mistakes give another answer on this data (sets, not only order)
    wrong_clamp = _normalised_choice_by_loop(flat_s, flat_p, limit, k, input_pos_after, prefill_len, clamp_shift=0)
    wrong_pos = _normalised_choice_by_loop(flat_s, flat_p, limit, k, input_pos_after, prefill_len, pos_shift=q_len)
    assert any(set(a) != set(b) for a, b in zip(want, wrong_clamp)), "data does not tell prefill_len from prefill_len - 1"
    assert any(set(a) != set(b) for a, b in zip(want, wrong_pos)), "data does not tell input_pos before from after the advance"


def test_normalised_cache_steps_against_a_per_token_model():
    """Cache level: which input_pos and which prefill length reach the division. The model keeps a
    dict token -> cumulative score per (b, h) and never sees a slot; after every step on a full cache
    the oracle's next_index, read back through its token positions, must be the tokens with the
    smallest score / (tokens seen so far, this step's included, - max(token, prefill_length - 1))."""
    B, Hq, Hkv, L, D, chunk = 1, 4, 2, 40, 8, 4
    n0 = 28  # prefill shorter than the cache: slots filled later are not clamped
    steps = (4, 4, 4, 3, 4, 1, 4, 2)
    q, k, v = _inputs(31, B, Hq, Hkv, n0 + sum(steps), D)
    ora = P.PolicyCacheOracle(B, Hq, Hkv, L, D, max_chunk_size=chunk, normalize_scores=True)
    ora.prefill(q[:, :, :n0], k[:, :, :n0], v[:, :, :n0])
    model = [[{t: 0.0 for t in range(n0)} for _ in range(Hkv)] for _ in range(B)]
    pos = n0
    checked = 0
    for num in steps:
        before_tp = ora.token_pos.clone()
        was_full = ora.current_length == L
        _, w, index = ora.forward(q[:, :, pos : pos + num], k[:, :, pos : pos + num], v[:, :, pos : pos + num])
        pos += num
        for b in range(B):
            for h in range(Hkv):
                m = model[b][h]
                if was_full:
                    for t in before_tp[b, h, index[b, h]].tolist():
                        del m[t]
                for t in range(pos - num, pos):
                    m[t] = 0.0
                tp = ora.token_pos[b, h, : ora.current_length].tolist()
                assert sorted(tp) == sorted(m)
                for slot, t in enumerate(tp):
                    m[t] = float(np.float32(m[t]) + np.float32(w[b, h, slot].item()))
                if ora.current_length == L:
                    ranked = sorted((np.float32(s) / np.float32(pos - max(t, n0 - 1)), tp.index(t)) for t, s in m.items())
                    kk = ora.next_index.shape[-1]
                    assert [slot for _, slot in ranked[:kk]] == ora.next_index[b, h].tolist()
                    checked += 1
    assert checked >= 4 * B * Hkv
