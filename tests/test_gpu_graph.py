"""The single-token serving step (slot write, then attention + score update + eviction choice in one
call) recorded once into a HIP graph through the C ABI and replayed: every replay consumes the slot
the replay before it chose. Between replays the program does eager work of its own and synchronises;
every replay is compared, bit for bit, with the same step launched eagerly on a second set of buffers.
Nothing in these entry points allocates, clears memory with a memset node or reads the host between
launches, which is what makes them recordable."""
import ctypes
import math

import pytest
import torch

from keys_values_amd import _lib
from keys_values_amd.attention import ops

pytestmark = pytest.mark.gpu


class _Step:
    """One cache (B, Hkv, L, D) in bf16 with its scores, positions, next slot and argument blocks."""

    def __init__(self, kvx, gpu, B, Hq, Hkv, L, D, seed):
        gen = torch.Generator().manual_seed(seed)
        self.kvx, self.gpu, self.L = kvx, gpu, L
        self.k = torch.randn(B, Hkv, L, D, generator=gen).to(torch.bfloat16).to(gpu)
        self.v = torch.randn(B, Hkv, L, D, generator=gen).to(torch.bfloat16).to(gpu)
        self.scores = (torch.rand(B, Hkv, L, generator=gen) * 2).to(gpu)
        self.token_pos = torch.arange(L, dtype=torch.int32).view(1, 1, L).expand(B, Hkv, L).contiguous().to(gpu)
        self.next_index = torch.zeros(B, Hkv, 1, dtype=torch.int32, device=gpu)
        # inputs of a step live in fixed buffers: a replay reads whatever they hold
        self.q = torch.zeros(B, Hq, 1, D, dtype=torch.bfloat16, device=gpu)
        self.nk = torch.zeros(B, Hkv, 1, D, dtype=torch.bfloat16, device=gpu)
        self.nv = torch.zeros(B, Hkv, 1, D, dtype=torch.bfloat16, device=gpu)
        self.out = torch.zeros(B, Hq, 1, D, dtype=torch.bfloat16, device=gpu)
        w = _lib.CacheWriteArgs()
        w.B, w.Hkv, w.num, w.D, w.cache_len = B, Hkv, 1, D, L
        w.input_pos, w.kv_dtype = L, _lib.KVX_KV_BF16  # the positions written are not read by this test
        w.index, w.index_stride_b, w.index_stride_h = self.next_index.data_ptr(), self.next_index.stride(0), self.next_index.stride(1)
        w.key, w.key_stride_b, w.key_stride_h, w.key_stride_t = self.nk.data_ptr(), self.nk.stride(0), self.nk.stride(1), self.nk.stride(2)
        w.value, w.value_stride_b, w.value_stride_h, w.value_stride_t = self.nv.data_ptr(), self.nv.stride(0), self.nv.stride(1), self.nv.stride(2)
        w.k_cache, w.kc_stride_b, w.kc_stride_h, w.kc_stride_t = self.k.data_ptr(), self.k.stride(0), self.k.stride(1), self.k.stride(2)
        w.v_cache, w.vc_stride_b, w.vc_stride_h, w.vc_stride_t = self.v.data_ptr(), self.v.stride(0), self.v.stride(1), self.v.stride(2)
        w.token_pos, w.tp_stride_b, w.tp_stride_h = self.token_pos.data_ptr(), self.token_pos.stride(0), self.token_pos.stride(1)
        w.scores, w.sc_stride_b, w.sc_stride_h = self.scores.data_ptr(), self.scores.stride(0), self.scores.stride(1)
        self.write_args = w
        a = _lib.SdpaArgs()
        ops._fill_common(a, self.q, self.k, self.v, 1.0 / math.sqrt(D), L - 1, None, None, 0)
        a.o, a.o_stride_b, a.o_stride_h, a.o_stride_t = self.out.data_ptr(), self.out.stride(0), self.out.stride(1), self.out.stride(2)
        h = _lib.H2OArgs()
        h.B, h.Hkv, h.kv_len, h.limit, h.k = B, Hkv, L, L, 1
        h.scores, h.sc_stride_b, h.sc_stride_h = self.scores.data_ptr(), self.scores.stride(0), self.scores.stride(1)
        h.next_index = self.next_index.data_ptr()
        nb_h = (kvx.kvx_h2o_workspace_bytes(ctypes.byref(h)) + 255) // 256 * 256
        nb_a = kvx.kvx_sdpa_decode_h2o_workspace_bytes(ctypes.byref(a))
        self.ws = torch.empty(nb_h + nb_a + 256, dtype=torch.uint8, device=gpu)
        h.workspace, h.workspace_bytes = self.ws.data_ptr(), nb_h
        a.workspace, a.workspace_bytes = self.ws.data_ptr() + nb_h, nb_a
        self.sdpa_args, self.h2o_args = a, h

    def launch(self):
        """The step's launches on the current stream."""
        stream = _lib.stream_ptr(self.gpu)
        _lib.check(self.kvx.kvx_cache_write(ctypes.byref(self.write_args), stream))
        _lib.check(self.kvx.kvx_sdpa_decode_h2o(ctypes.byref(self.sdpa_args), ctypes.byref(self.h2o_args), stream))

    def feed(self, q, nk, nv):
        self.q.copy_(q)
        self.nk.copy_(nk)
        self.nv.copy_(nv)

    def state(self):
        return [t.clone() for t in (self.out, self.scores, self.next_index, self.k, self.v)]


@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(2, 8, 2, 6000, 128), (1, 6, 2, 777, 64)])
def test_decode_step_replayed_from_a_graph(kvx, gpu, decode_route, B, Hq, Hkv, L, D):
    eager = _Step(kvx, gpu, B, Hq, Hkv, L, D, seed=31)
    replayed = _Step(kvx, gpu, B, Hq, Hkv, L, D, seed=31)
    gen = torch.Generator().manual_seed(32)
    steps = [tuple(torch.randn(B, h, 1, D, generator=gen).to(torch.bfloat16).to(gpu) for h in (Hq, Hkv, Hkv)) for _ in range(6)]
    # one eager step on both (the first call on a device also looks its properties up), then record
    for s in (eager, replayed):
        s.feed(*steps[0])
        s.launch()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream(gpu)
    replayed.feed(*steps[1])
    eager.feed(*steps[1])
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        replayed.launch()  # recorded, not run
    busy = torch.randn(512, 512, device=gpu)
    for i in range(1, 6):
        for s in (eager, replayed):
            s.feed(*steps[i])
        eager.launch()
        graph.replay()
        busy = (busy @ busy).clamp_(-1, 1)  # the program's own eager work between the replays
        torch.cuda.synchronize()
        for x, y in zip(eager.state(), replayed.state()):
            assert torch.equal(x, y), f"replay {i}"
    assert (replayed.next_index >= 0).all() and (replayed.next_index < L).all()
