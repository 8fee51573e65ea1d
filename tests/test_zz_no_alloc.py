"""kvx_h2o_update_select_static (the entry point that allocates nothing: its scratch is a device array
inside the library) against kvx_h2o_update_select on the same inputs, through the C ABI. Two calls in
a row share the array, the second on a smaller input; then the policy variant that keeps per-row
statistics in the scratch, and the size limit."""
import ctypes

import pytest
import torch

from keys_values_amd import _lib

pytestmark = pytest.mark.gpu


def _args(gpu, scores, w, k, next_index, token_pos=None, normalize=False, input_pos=0, prefill_len=0, q_errors=None, combination=0.0):
    B, Hkv, L = scores.shape
    a = _lib.H2OArgs()
    a.B, a.Hkv, a.kv_len, a.limit, a.k = B, Hkv, L, L, k
    a.normalize, a.input_pos, a.prefill_len = int(normalize), input_pos, prefill_len
    a.scores, a.sc_stride_b, a.sc_stride_h = scores.data_ptr(), scores.stride(0), scores.stride(1)
    a.w = _lib.ptr(w)
    if token_pos is not None:
        a.token_pos, a.tp_stride_b, a.tp_stride_h = token_pos.data_ptr(), token_pos.stride(0), token_pos.stride(1)
    a.next_index = next_index.data_ptr()
    if q_errors is not None:
        a.q_errors, a.combination = q_errors.data_ptr(), combination
    return a


def _both(kvx, gpu, scores, w, k, **kw):
    """(scores, next) of the entry point with a caller workspace and of the static one."""
    B, Hkv, L = scores.shape
    out = []
    for static in (False, True):
        sc = scores.clone()
        nxt = torch.full((B, Hkv, k), -1, dtype=torch.int32, device=gpu)
        a = _args(gpu, sc, w, k, nxt, **kw)
        if static:
            a.workspace, a.workspace_bytes = None, 0
            print(f"static call B={B} Hkv={Hkv} L={L} k={k}", flush=True)
            _lib.check(kvx.kvx_h2o_update_select_static(ctypes.byref(a), _lib.stream_ptr(gpu)))
        else:
            nb = kvx.kvx_h2o_workspace_bytes(ctypes.byref(a))
            ws = torch.empty(max(nb, 16), dtype=torch.uint8, device=gpu)
            a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
            _lib.check(kvx.kvx_h2o_update_select(ctypes.byref(a), _lib.stream_ptr(gpu)))
        torch.cuda.synchronize()
        out.append((sc.cpu(), nxt.cpu()))
    return out


def test_static_scratch_matches_workspace_entry_point(kvx, gpu):
    gen = torch.Generator().manual_seed(11)
    # two calls in a row on the shared array, the second smaller (fewer rows, shorter rows), k = 1 uses the
    # scratch for the per-row minimum keys
    for B, Hkv, L, k in ((8, 8, 20000, 1), (2, 3, 777, 1), (2, 2, 5000, 256), (1, 2, 300, 7)):
        scores = (torch.rand(B, Hkv, L, generator=gen) * 3).to(gpu)
        w = torch.rand(B, Hkv, L, generator=gen).to(gpu)
        (s0, n0), (s1, n1) = _both(kvx, gpu, scores, w, k)
        assert torch.equal(s0, s1), (B, Hkv, L, k)
        assert torch.equal(n0, n1), (B, Hkv, L, k)
        assert (n1 >= 0).all() and (n1 < L).all()
        assert torch.equal(s0, (scores + w).cpu())


def test_static_scratch_policy_statistics(kvx, gpu):
    # the q_errors combination keeps four numbers per row in the scratch, next to the minimum keys
    gen = torch.Generator().manual_seed(12)
    for B, Hkv, L, k in ((4, 8, 3000, 1), (2, 2, 600, 1), (1, 4, 900, 33)):
        scores = (torch.rand(B, Hkv, L, generator=gen) * 3).to(gpu)
        w = torch.rand(B, Hkv, L, generator=gen).to(gpu)
        qe = torch.rand(B, Hkv, L, generator=gen).to(gpu)
        tp = torch.stack([torch.randperm(4000, generator=gen)[:L] for _ in range(B * Hkv)]).view(B, Hkv, L).to(torch.int32).to(gpu)
        (s0, n0), (s1, n1) = _both(kvx, gpu, scores, w, k, token_pos=tp, normalize=True, input_pos=4100, prefill_len=512, q_errors=qe, combination=0.7)
        assert torch.equal(s0, s1) and torch.equal(n0, n1), (B, Hkv, L, k)


def test_static_scratch_rejects_what_does_not_fit(kvx, gpu):
    # 128 KiB / 8 bytes per row: more rows than that cannot keep their minimum keys in the array
    B, Hkv, L = 4100, 4, 8
    scores = torch.zeros(B, Hkv, L, device=gpu)
    nxt = torch.zeros(B, Hkv, 1, dtype=torch.int32, device=gpu)
    a = _args(gpu, scores, None, 1, nxt)
    assert kvx.kvx_h2o_workspace_bytes(ctypes.byref(a)) > 128 * 1024
    rc = kvx.kvx_h2o_update_select_static(ctypes.byref(a), _lib.stream_ptr(gpu))
    assert rc == _lib.KVX_ERR_WORKSPACE and b"static array holds" in kvx.kvx_last_error()
    torch.cuda.synchronize()
