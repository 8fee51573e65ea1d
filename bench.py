#!/usr/bin/env python3
"""
Benchmark of the attention-with-score-sums hot path on one MI355X.

Default workload (`--workload prefill`): the Qwen3-4B-shaped chunked prefill of BASELINE.json
(batch 1, 32 query / 8 KV heads, head size 128, 32768 cached positions, a 1024-query chunk appended
causally at the end, bf16, RoPE theta 1e6, seed 1). One step = attention output + base-2 LSE +
per-key score-sums for the whole chunk: the prefill kernel followed by the score-sum kernel.
Inputs are resident in HBM before the timed region.

`--workload decode`  : single-token decode over a bf16 cache with score-sums, H2O score update and
                       argmin (batch 8, 32/8 heads, 131072 positions), GB/s against HBM peak.
`--workload quantize`: affine uint8 row quantiser on (1, 8, 65536, 128) K and V, GB/s.
`--workload longctx` : BASELINE.json configs[4]: random-init Qwen3-4B-shaped stack (36 layers), 131072 random
                       tokens in chunks of 1024 after a 16384-token first chunk, uint8 H2O caches of 16384
                       slots per layer; end-to-end prefill tokens/s. One step = one whole sequence.
                       `--layers N --tokens T` shrink it (stated in the output); `--tune-gemms` lets the GEMM
                       library choose its kernels by measurement during the warm-up pass.
`--workload policy`  : the same 1024-token chunk through the cache object (write with the ring move, attention,
                       score-sum, score update, choice of the next 1024 slots) for each eviction-policy variant
                       (grace period, normalised scores, V-norm weighting, Q-Hitter); ms per chunk step.
`--workload calib`   : a plain elementwise kernel that reads 1 GiB and writes 1 GiB, the known-size
                       launch against which the FETCH_SIZE / WRITE_SIZE counters are scaled.

The default run also times, after the headline workload, the decode + H2O step, the quantiser, attention +
score-sum over the uint8 store (BASELINE.json configs[2]: fused dequantisation and the dequantised-copy path) and the
long-context prefill on their own configurations and reports them under `config.secondary`
(`--no-secondary` skips them).

Prints ONE JSON line (see the keys below). `roofline` describes the dominant kernel, timed with
events on the launch stream inside the timed steps; `cpu_baseline` times the CPU oracle (the
reference's eager op sequence restated) on a bounded sample of the same workload.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E

# HBM bytes per launch of each workload's dominant kernel. NOT measured by this run: the figures of the
# committed counter runs (profiles/hbm_traffic_fetch_write_size.txt: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE,
# KiB per dispatch, one counter per run, on these same workloads), each scaled by what the counter reads for
# the `calib` launch of known size (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000). Reported as `roofline.traffic`
# with `roofline.traffic_source` saying so. (The quantiser's 2 x 205 MB working set is close to the 256 MB
# last-level cache; its FETCH_SIZE still reads the full 134 MB per launch, so the rows do come from HBM.)
TRAFFIC_SOURCE = "committed counter run (profiles/hbm_traffic_fetch_write_size.txt), not measured in this run"
TRAFFIC_BYTES = {
    "prefill": int((70196.3 * 2.000 + 33283.4) * 1024),    # sdpa_prefill_kernel<128, KVX_KV_BF16>
    "decode": int((2115128.0 * 2.000 + 37312.0) * 1024),   # decode_split_kernel<128, 4, KVX_KV_BF16>
    "quantize": int((65573.9 * 2.000 + 69632.0) * 1024),   # quantize_rows_kernel<128>
}


def cpu_threads(torch):
    """Threads for the CPU baseline: the GPU box's share of host cores is 16 per GPU whatever os.cpu_count() shows
    there, so more threads than that would only time-slice."""
    n = min(16, os.cpu_count() or 1)
    torch.set_num_threads(n)
    return n


def cpu_time(fn):
    """Seconds of one pass of `fn`: the median of 5 passes when a pass takes at most 2 s (after the first pass, which
    then counts as the warm-up), else that single pass. Returns (seconds, result of the last pass, note)."""
    t0 = time.perf_counter()
    res = fn()
    first = time.perf_counter() - t0
    if first > 2.0:
        return first, res, "one pass"
    ts = []
    for _ in range(5):
        t0 = time.perf_counter()
        res = fn()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    return ts[len(ts) // 2], res, "median of 5 passes after 1 warm-up"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="prefill", choices=["prefill", "decode", "quantize", "longctx", "policy", "calib"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="default workload only: skip the decode, quantiser and long-context legs that are reported under config.secondary")
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--layers", type=int, default=36, help="longctx: number of layers")
    ap.add_argument("--tokens", type=int, default=131072, help="longctx: prompt length")
    ap.add_argument("--no-gemm-table", action="store_true",
                    help="longctx: leave the choice of the library GEMM kernels to the library instead of reading the committed per-shape "
                         "table (keys_values_amd/longctx/gemm_table_gfx950.csv; switches PyTorch's TunableOp on for the process)")
    ap.add_argument("--tune-gemms", action="store_true",
                    help="longctx: let PyTorch's TunableOp pick the library GEMM kernels during the warm-up pass (adds about a minute)")
    ap.add_argument("--operands", default="random", choices=["random", "zeros"],
                    help="prefill: `zeros` runs the same launches on all-zero q, k, v (not the benchmark: a probe of how much of the "
                         "duration is the clock following the operands; the line says so in `data`)")
    ap.add_argument("--kv", default="bf16", choices=["bf16", "uint8", "uint4"],
                    help="cache storage for the prefill / decode workloads; uint8 = BASELINE.json configs[2]: codes + per-row "
                         "scale and zero point, dequantised inside the attention kernels; uint4 = the 4-bit store of the same quantiser")
    return ap.parse_args()


def rope_inputs(torch, O, dev, T=32768, seed=1, zeros=False):
    B, Hq, Hkv, q_len, D = 1, 32, 8, 1024, 128
    input_pos = T - q_len
    if zeros:  # the same launches on operands that toggle nothing: what the clock does without the data's share of the power
        z = lambda *shape: torch.zeros(shape, dtype=torch.bfloat16)
        return (B, Hq, Hkv, q_len, T, D, input_pos), z(B, Hq, q_len, D), z(B, Hkv, T, D), z(B, Hkv, T, D)
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, q_len, D, generator=gen)
    k = torch.randn(B, Hkv, T, D, generator=gen)
    v = torch.randn(B, Hkv, T, D, generator=gen).to(torch.bfloat16)
    q = O.apply_rope(q, torch.arange(input_pos, input_pos + q_len)).to(torch.bfloat16)
    k = O.apply_rope(k, torch.arange(T)).to(torch.bfloat16)
    return (B, Hq, Hkv, q_len, T, D, input_pos), q, k, v


def bench_prefill(args, torch, dev):
    from keys_values_amd import _lib
    from keys_values_amd.attention import ops
    from oracle import kvx_oracle as O

    lib = _lib.load()
    u8 = args.kv != "bf16"   # a quantised store: codes + row state
    u4 = args.kv == "uint4"
    (B, Hq, Hkv, q_len, T, D, input_pos), q_c, k_c, v_c = rope_inputs(torch, O, dev, 65536 if u8 else 32768, 2 if u8 else 1, args.operands == "zeros")
    scale = D ** -0.5
    q, k, v = q_c.to(dev), k_c.to(dev), v_c.to(dev)
    quant = None
    if u8:
        # quantise with the library's own kernel; the CPU sample below attends over the dequantised rows
        def quantise(x):
            c = torch.empty(x.shape[:-1] + (D // 2 if u4 else D,), dtype=torch.uint8, device=dev)
            sc = torch.empty(x.shape[:-1], dtype=torch.float32, device=dev)
            zp = torch.empty(x.shape[:-1], dtype=torch.int32, device=dev)
            fn = lib.kvx_quantize_rows4 if u4 else lib.kvx_quantize_rows
            _lib.check(fn(x.data_ptr(), D, x.numel() // D, D, c.data_ptr(), sc.data_ptr(), zp.data_ptr(), _lib.stream_ptr(dev)))
            return c, sc, zp
        k, ksc, kzp = quantise(k)
        v, vsc, vzp = quantise(v)
        quant = ops.QuantState(ksc, kzp, vsc, vzp)
        torch.cuda.synchronize()
        unpack = O.uncompress4 if u4 else (lambda c: c)
        k_c = O.dequantize_rows(unpack(k.cpu()), ksc.cpu(), kzp.cpu())
        v_c = O.dequantize_rows(unpack(v.cpu()), vsc.cpu(), vzp.cpu())
    out = torch.empty((B, q_len, Hq, D), dtype=torch.bfloat16, device=dev)
    o_view = out.permute(0, 2, 1, 3)
    lse = torch.empty((B, q_len, Hq), dtype=torch.float32, device=dev)
    w = torch.empty((B, Hkv, T), dtype=torch.float32, device=dev)
    a = _lib.SdpaArgs()
    ops._fill_common(a, q, k, v, scale, input_pos, None, quant, args.splits)
    a.o = o_view.data_ptr()
    a.o_stride_b, a.o_stride_h, a.o_stride_t = o_view.stride(0), o_view.stride(1), o_view.stride(2)
    a.lse, a.w = lse.data_ptr(), w.data_ptr()
    nbytes = lib.kvx_sdpa_prefill_workspace_bytes(ctypes.byref(a))
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    st = _lib.stream_ptr(dev)

    def step(ev=None):
        if ev is not None:
            ev[0].record()
        _lib.check(lib.kvx_sdpa_prefill(ctypes.byref(a), st))
        if ev is not None:
            ev[1].record()
        _lib.check(lib.kvx_score_sum(ctypes.byref(a), st))
        if ev is not None:
            ev[2].record()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_step = (t1 - t0) * 1e3 / args.steps
    ms_attn = sum(e[0].elapsed_time(e[1]) for e in events) / args.steps
    ms_score = sum(e[1].elapsed_time(e[2]) for e in events) / args.steps

    flops_alg = 4.0 * B * Hq * q_len * T * D        # QK^T + PV: credited for O, LSE and W together
    flops_issued = 6.0 * B * Hq * q_len * T * D     # the score-sum pass repeats QK^T
    tflops = flops_alg / (ms_step * 1e-3) / 1e12
    attn_tflops = flops_alg / (ms_attn * 1e-3) / 1e12

    # sanity of the timed outputs (cheap invariants; the parity tests do the real checking)
    rows = w.sum(-1).cpu()
    assert torch.allclose(rows, torch.full_like(rows, float(q_len)), rtol=1e-4, atol=5e-2), rows

    # A quantised store, long chunk: what the cache object does instead of dequantising inside the attention
    # kernels (where every workgroup of 256 rows dequantises the whole store again) is one dequantisation
    # of the store into a bf16 copy for the attention kernel (the score-sum kernel dequantises each key once
    # per wavefront anyway and stays on the codes). Timed here on the same inputs.
    dq_ms = None
    if u8:
        from keys_values_amd.kvcache.h2o import _dequant_scratch

        kd, vd, _ = _dequant_scratch(dev, B * Hkv * T * D)  # the cache object's own buffer
        kd, vd = kd.view(B, Hkv, T, D), vd.view(B, Hkv, T, D)
        dq = lib.kvx_dequantize_rows4 if u4 else lib.kvx_dequantize_rows

        def step_copy():
            _lib.check(dq(k.data_ptr(), ksc.data_ptr(), kzp.data_ptr(), B * Hkv * T, D, kd.data_ptr(), D, st))
            _lib.check(dq(v.data_ptr(), vsc.data_ptr(), vzp.data_ptr(), B * Hkv * T, D, vd.data_ptr(), D, st))
            _, _, lse_c = ops.prefill_core(q, kd, vd, scale, input_pos, None, return_lse=True)
            return ops.score_sum_core(q, k, lse_c, scale, input_pos, None, quant=quant)  # the score-sum pass keeps the codes

        for _ in range(3):
            w_copy = step_copy()
        torch.cuda.synchronize()
        torch.testing.assert_close(w_copy, w, rtol=1e-3, atol=1e-6)
        d0, d1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        d0.record()
        for _ in range(10):
            step_copy()
        d1.record()
        torch.cuda.synchronize()
        dq_ms = d0.elapsed_time(d1) / 10

    # The same chunk through the cache object (keys_values/kvcache/base.py:554-595): write the 1024 new
    # rows into the slots chosen by the step before, attend, score-sum, scores += W, choose the next
    # 1024 lowest-score slots. Steady state: after the first step the positions are scattered.
    h2o_ms = None
    if not u8:
        from keys_values_amd.kvcache.h2o import H2OKVCache, KVCacheParams
        cache = H2OKVCache(KVCacheParams(B, Hkv, T, D, Hq), max_chunk_size=q_len, device=dev)
        cache.k.copy_(k)
        cache.v.copy_(v)
        cache.token_pos.copy_(torch.arange(T, dtype=torch.int32, device=dev).view(1, 1, T).expand(B, Hkv, T))
        cache.scores.copy_(torch.rand((B, Hkv, T), device=dev))
        cache.batch_size, cache.current_length, cache.prefill_length = B, T, T
        cache._input_pos = T
        cache._use_initial_rule = False
        cache.set_next_positions(torch.arange(q_len, dtype=torch.int32, device=dev).view(1, 1, q_len).expand(B, Hkv, q_len))
        kn, vn = k[:, :, -q_len:].contiguous(), v[:, :, -q_len:].contiguous()
        for _ in range(3):
            cache.forward(q, kn, vn)
        torch.cuda.synchronize()
        h0, h1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        h0.record()
        for _ in range(10):
            cache.forward(q, kn, vn)
        h1.record()
        torch.cuda.synchronize()
        h2o_ms = h0.elapsed_time(h1) / 10

    cpu = None
    if not args.no_cpu_baseline:
        # bounded sample: the first KV heads with their query heads, same op sequence as the
        # reference's eager path (fp32 upcast, <= 3 GB score slices, mask, softmax, mean/sum)
        nthreads = cpu_threads(torch)
        hs = 1 if u8 else Hkv  # bf16: the whole workload, a second or two on the host's cores; quantised store: one KV head
        qs, ks, vs = q_c[:, : 4 * hs], k_c[:, :hs], v_c[:, :hs]
        t_c, (o_ref, w_ref), how = cpu_time(lambda: O.sdpa_in_blocks(qs, ks, vs, scale, input_pos, None))
        cpu = {
            "value": round(flops_alg * hs / Hkv / t_c / 1e12, 4),
            "unit": "TFLOP/s",
            "cores": nthreads,
            "host_cpus": os.cpu_count(),
            "kind": "port",
            "sample": f"KV heads 0-{hs - 1} of {Hkv} ({4 * hs} query heads x 1024 queries x {T} keys"
                      + (", over the dequantised rows" if u8 else "") + f"), {how}, {t_c:.2f} s a pass",
        }
        # the sample doubles as an end-to-end check of the timed outputs
        err = ((out.permute(0, 2, 1, 3)[:, : 4 * hs].float().cpu() - o_ref.float()).norm() / o_ref.float().norm()).item()
        assert err < 2e-2, err
        torch.testing.assert_close(w[:, :hs].cpu(), w_ref, rtol=1e-3, atol=1e-6)

    return {
        "metric": "attn+score-sum TFLOP/s (% MFMA peak); H2O prefill tok/s, Qwen3-4B shape",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic" if args.operands == "random" else "synthetic, ALL-ZERO operands (clock probe, not the benchmark)",
        "config": {
            "workload": (f"BASELINE.json configs[2]: attention + score-sum over the {args.kv} cache (dequantised in the kernels), B1 Hq32 Hkv8 D128 T65536 q1024, seed 2"
                         if u8 else
                         "BASELINE.json configs[1]: chunked prefill attention + score-sum, B1 Hq32 Hkv8 D128 T32768 q1024, RoPE theta 1e6, seed 1"),
            "flops_algorithmic": flops_alg,
            "flops_issued": flops_issued,
            "pct_mfma_peak": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
            "chunk_tokens_per_s": round(q_len / (ms_step * 1e-3), 1),
            "ms_attention_kernel": round(ms_attn, 4),
            "ms_score_sum_kernel": round(ms_score, 4),
            "score_sum_tflops": round(2.0 * B * Hq * q_len * T * D / (ms_score * 1e-3) / 1e12, 2),
            "ms_step_over_dequantised_copy": None if dq_ms is None else round(dq_ms, 4),
            "h2o_cache_chunk_ms": None if h2o_ms is None else round(h2o_ms, 4),
            "h2o_cache_chunk_tokens_per_s": None if h2o_ms is None else round(q_len / (h2o_ms * 1e-3), 1),
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "sdpa_prefill_kernel<128,%s> (+ split merge)" % {"bf16": "KVX_KV_BF16", "uint8": "KVX_KV_U8", "uint4": "KVX_KV_U4"}[args.kv],
            "achieved": round(attn_tflops, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(attn_tflops / PEAK_BF16_TFLOPS, 4),
            "traffic": None if u8 else TRAFFIC_BYTES["prefill"],
            "traffic_source": None if u8 else TRAFFIC_SOURCE,
        },
        "cpu_baseline": cpu,
    }


def bench_quantize(args, torch, dev):
    from keys_values_amd import _lib
    from oracle import kvx_oracle as O

    lib = _lib.load()
    rows, D = 8 * 65536, 128
    gen = torch.Generator().manual_seed(2)
    kx = torch.randn(rows, D, generator=gen)
    mask = torch.rand(rows, D, generator=gen) < 0.01
    kx = torch.where(mask, torch.randn(rows, D, generator=gen) * 8, kx).to(torch.bfloat16)
    vx = torch.randn(rows, D, generator=gen).to(torch.bfloat16)
    xs = [kx.to(dev), vx.to(dev)]
    outs = [(torch.empty((rows, D), dtype=torch.uint8, device=dev), torch.empty(rows, dtype=torch.float32, device=dev),
             torch.empty(rows, dtype=torch.int32, device=dev)) for _ in xs]
    st = _lib.stream_ptr(dev)

    def step():
        for x, (c, s, z) in zip(xs, outs):
            _lib.check(lib.kvx_quantize_rows(x.data_ptr(), D, rows, D, c.data_ptr(), s.data_ptr(), z.data_ptr(), st))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_kernel = e0.elapsed_time(e1) / args.steps / 2
    bytes_alg = rows * (2 * D + D + 8)  # per tensor: bf16 in, codes + fp32 scale + int32 zero point out
    gbs = 2 * bytes_alg / (ms_step * 1e-3) / 1e9
    kgbs = bytes_alg / (ms_kernel * 1e-3) / 1e9
    cpu = None
    if not args.no_cpu_baseline:
        nthreads = cpu_threads(torch)
        t_c, (c_ref, s_ref, z_ref), how = cpu_time(lambda: O.quantize_rows(kx))
        cpu = {"value": round(bytes_alg / t_c / 1e9, 3), "unit": "GB/s", "cores": nthreads, "host_cpus": os.cpu_count(), "kind": "port",
               "sample": f"K tensor only (half the workload), {how}, {t_c:.2f} s a pass"}
        assert torch.equal(outs[0][0].cpu(), c_ref) and torch.equal(outs[0][1].cpu(), s_ref) and torch.equal(outs[0][2].cpu(), z_ref)
    return {
        "metric": "uint8 row quantiser GB/s (% HBM peak)", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[2] quantiser: K and V (1, 8, 65536, 128) bf16 -> uint8 + fp32 scale + int32 zero point, seed 2",
                   "bytes_algorithmic_per_tensor": bytes_alg},
        "roofline": {"bound": "hbm", "kernel": "quantize_rows_kernel<128>", "achieved": round(kgbs, 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(kgbs / PEAK_HBM_GBS, 4), "traffic": TRAFFIC_BYTES["quantize"], "traffic_source": TRAFFIC_SOURCE},
        "cpu_baseline": cpu,
    }


def bench_decode(args, torch, dev):
    from keys_values_amd import _lib
    from keys_values_amd.kvcache.h2o import H2OKVCache, KVCacheParams
    from oracle import kvx_oracle as O

    B, Hq, Hkv, L, D = 8, 32, 8, 131072, 128
    gen = torch.Generator(device=dev).manual_seed(3)
    u8 = args.kv != "bf16"
    u4 = args.kv == "uint4"
    cache = H2OKVCache(KVCacheParams(B, Hkv, L, D, Hq), max_chunk_size=1, quantized=u8, num_bits=4 if u4 else 8, device=dev)
    # state as after a prefill that filled the cache (the prefill itself is not part of this workload)
    if u8:
        lib = _lib.load()
        for codes, sc, zp in ((cache.k, cache.k_scale, cache.k_zp), (cache.v, cache.v_scale, cache.v_zp)):
            for bi in range(B):  # one batch row at a time keeps the bf16 temporaries small
                x = torch.randn((Hkv, L, D), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
                fn = lib.kvx_quantize_rows4 if u4 else lib.kvx_quantize_rows
                _lib.check(fn(x.data_ptr(), D, x.numel() // D, D, codes[bi].data_ptr(), sc[bi].data_ptr(),
                              zp[bi].data_ptr(), _lib.stream_ptr(dev)))
            torch.cuda.synchronize()
    else:
        cache.k.copy_(torch.randn(cache.k.shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16))
        cache.v.copy_(torch.randn(cache.v.shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16))
    cache.token_pos.copy_(torch.arange(L, dtype=torch.int32, device=dev).view(1, 1, L).expand(B, Hkv, L))
    cache.batch_size, cache.current_length, cache.prefill_length = B, L, L
    cache._input_pos = L
    cache._use_initial_rule = False
    cache.set_next_positions(torch.zeros((B, Hkv, 1), dtype=torch.int32, device=dev))
    n = args.steps + args.warmup
    qs = torch.randn((n, B, Hq, 1, D), generator=gen, device=dev).to(torch.bfloat16)
    ks = torch.randn((n, B, Hkv, 1, D), generator=gen, device=dev).to(torch.bfloat16)
    vs = torch.randn((n, B, Hkv, 1, D), generator=gen, device=dev).to(torch.bfloat16)
    for i in range(args.warmup):
        cache.forward(qs[i], ks[i], vs[i])
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(args.warmup, n):
        cache.forward(qs[i], ks[i], vs[i])
    e1.record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_gpu = e0.elapsed_time(e1) / args.steps
    # K + V once (bf16 rows, or codes + 8 bytes of row state), scores read-modify-write
    bytes_alg = 2 * B * Hkv * L * ((D // 2 if u4 else D) + 8 if u8 else 2 * D) + 2 * B * Hkv * L * 4
    gbs = bytes_alg / (ms_step * 1e-3) / 1e9
    # the dominant launch alone: the fused attention + score update + argmin call (split attention,
    # tail kernel), events on the launch stream around each call
    launch, _ = cache._decode_h2o_prepare(qs[0], cache.k, cache.v, cache._quant_state(L))
    launch()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a0, a1 in evs:
        a0.record()
        launch()
        a1.record()
    torch.cuda.synchronize()
    ms_call = sum(a0.elapsed_time(a1) for a0, a1 in evs) / args.steps
    cpu = None
    if not args.no_cpu_baseline:
        nthreads = cpu_threads(torch)
        nb = B  # the attention of one whole step
        if u8:
            unpack = O.uncompress4 if u4 else (lambda c: c)
            kc = O.dequantize_rows(unpack(cache.k[:nb].cpu()), cache.k_scale[:nb].cpu(), cache.k_zp[:nb].cpu())
            vc = O.dequantize_rows(unpack(cache.v[:nb].cpu()), cache.v_scale[:nb].cpu(), cache.v_zp[:nb].cpu())
        else:
            kc, vc = cache.k[:nb].cpu(), cache.v[:nb].cpu()
        qc = qs[0, :nb].cpu()
        t_c, _, how = cpu_time(lambda: O.sdpa_in_blocks(qc, kc, vc, D ** -0.5, L, None))
        frac = nb / B
        cpu = {"value": round(bytes_alg * frac / t_c / 1e9, 3), "unit": "GB/s", "cores": nthreads, "host_cpus": os.cpu_count(), "kind": "port",
               "sample": f"attention + score-sums of one step for batch rows 0-{nb - 1} of {B} ({frac:.2f} of a step), {how}, {t_c:.2f} s a pass"}
    return {
        "metric": "decode + H2O step GB/s (% HBM peak)", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[3]: decode + H2O eviction, B8 Hq32 Hkv8 D128 T131072, seed 3" + (f", {args.kv} cache" if u8 else ""),
                   "bytes_algorithmic_per_step": bytes_alg, "ms_per_step_gpu_events": round(ms_gpu, 4),
                   "decode_tokens_per_s": round(B / (ms_step * 1e-3), 1)},
        "roofline": {"bound": "hbm", "kernel": "kvx_sdpa_decode_h2o: decode_split_kernel<128,4,%s> + tail (merge, scratch-route weights, slot publishing)" % {"bf16": "KVX_KV_BF16", "uint8": "KVX_KV_U8", "uint4": "KVX_KV_U4"}[args.kv],
                     "achieved": round(bytes_alg / (ms_call * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(bytes_alg / (ms_call * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "ms_per_launch": round(ms_call, 4),
                     "traffic": None if u8 else TRAFFIC_BYTES["decode"], "traffic_source": None if u8 else TRAFFIC_SOURCE},
        "cpu_baseline": cpu,
    }


def bench_longctx(args, torch, dev):
    import dataclasses

    from keys_values_amd.longctx.model import QWEN3_4B, LongContextPrefillModel

    cfg = dataclasses.replace(QWEN3_4B, n_layer=args.layers)
    L, chunk, seq = 16384, 1024, args.tokens
    model = LongContextPrefillModel(cfg, cache_length=L, chunk_size=chunk, max_batch_size=1, quantized=True, max_context=max(seq, L), seed=4,
                                    device=dev, gemm_table=not args.no_gemm_table)
    ids = torch.randint(0, cfg.vocab_size, (1, seq), generator=torch.Generator().manual_seed(4))
    sizes = model.chunk_sizes(seq)
    steps = max(1, min(args.steps, 3))
    warm = 1 if args.warmup > 0 else 0
    if args.tune_gemms:  # the linear layers are plain library GEMMs: which kernel serves each shape is the library's choice
        import torch.cuda.tunable as tunable

        tunable.enable(True)
        tunable.tuning_enable(True)
        tunable.set_max_tuning_duration(15)
        tunable.set_max_tuning_iterations(20)
        tunable.set_filename(os.path.join(tempfile.gettempdir(), "kvx_bench_tunableop.csv"))  # its results file: not into the tree
        warm = 1
    for _ in range(warm):
        model.prefill(ids)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        h = model.prefill(ids)
    e1.record()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    ms_gpu = e0.elapsed_time(e1) / steps
    assert torch.isfinite(h.float()).all()
    # algorithmic FLOP: attention + score-sums per chunk and layer, causal first chunk, dense layers
    Hq, D = cfg.n_head, cfg.head_size
    attn = 0.0
    for i, n in enumerate(sizes):
        T = min(sum(sizes[: i + 1]), L)
        attn += (2.0 * Hq * n * n * D) if i == 0 else (4.0 * Hq * n * T * D)
    attn *= cfg.n_layer
    per_tok = 2.0 * cfg.n_layer * (cfg.n_embd * (Hq + 2 * cfg.n_query_groups) * D + Hq * D * cfg.n_embd + 3 * cfg.n_embd * cfg.intermediate_size)
    dense = per_tok * seq
    cpu = None
    if not args.no_cpu_baseline:
        # bounded sample: one layer, the first chunk shortened to 2048 tokens plus two 1024-token chunks on a
        # 2048-slot cache, through the CPU oracle of the same stack (same op sequence as the reference's eager path)
        from oracle import longctx_oracle as LO

        nthreads = cpu_threads(torch)
        c1 = dataclasses.replace(cfg, n_layer=1)
        layer = model.layers[0]
        weights = [{k: getattr(layer, k).cpu() for k in ("qkv", "proj", "fc_1", "fc_2", "mlp_proj", "norm_1", "norm_2", "norm_q", "norm_k")}]
        ref = LO.PrefillOracle(c1, model.wte.cpu(), weights, model.ln_f.cpu(), 2048, chunk, 1, True, 4096)
        t_c0 = time.perf_counter()
        ref.forward_chunk(ids[:, :2048])
        ref.forward_chunk(ids[:, 2048:3072])
        ref.forward_chunk(ids[:, 3072:4096])
        t_c = time.perf_counter() - t_c0
        cpu = {"value": round(4096 / t_c / cfg.n_layer, 2), "unit": "tokens/s", "cores": nthreads, "host_cpus": os.cpu_count(), "kind": "port",
               "sample": f"one layer over 4096 tokens (2048-token first chunk, two 1024-token chunks, 2048-slot cache) in {t_c:.1f} s, "
                         f"scaled to {cfg.n_layer} layers"}
    tps = seq / (ms_step * 1e-3)
    return {
        "metric": "H2O long-context prefill tokens/s, Qwen3-4B shape", "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warm, "ms_per_step": round(ms_step, 2), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"BASELINE.json configs[4]: random-init Qwen3-4B-shaped stack, {cfg.n_layer} layers, {seq} random tokens, "
                               f"chunks {sizes[0]} + {len(sizes) - 1} x {chunk}, uint8 H2O caches of {L} slots, seed 4",
                   "ms_per_step_gpu_events": round(ms_gpu, 2), "flops_attention_score_sums": attn, "flops_dense_layers": dense,
                   "tflops_total": round((attn + dense) / (ms_step * 1e-3) / 1e12, 1), "library_gemms": "tuned (TunableOp)" if args.tune_gemms else ("committed per-shape table" if model.gemm_table else "library default")},
        "roofline": {"bound": "mfma", "kernel": "whole prefill (attention + score-sum kernels and library GEMMs)",
                     "achieved": round((attn + dense) / (ms_gpu * 1e-3) / 1e12, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round((attn + dense) / (ms_gpu * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4), "traffic": None},
        "cpu_baseline": cpu,
    }


def bench_policy(args, torch, dev):
    """One 1024-token chunk into a full 32768-slot cache, per policy variant, through the cache object."""
    from keys_values_amd.kvcache.h2o import KVCacheParams, create_kv_cache
    from oracle import kvx_oracle as O

    (B, Hq, Hkv, q_len, T, D, input_pos), q_c, k_c, v_c = rope_inputs(torch, O, dev)
    q, k, v = q_c.to(dev), k_c.to(dev), v_c.to(dev)
    kn, vn = k[:, :, -q_len:].contiguous(), v[:, :, -q_len:].contiguous()
    variants = [
        ("h2o-default", dict()),
        ("h2o-default", dict(grace_period=256)),
        ("h2o-default", dict(grace_period=256, normalize_scores=True)),
        ("h2o-vlen-default", dict(grace_period=256)),
        ("h2o-torch-quantized8", dict(grace_period=256)),
        ("qh2o-torch-quantized8", dict(grace_period=256)),
        ("qh2o-vlen-torch-quantized8", dict(grace_period=256, normalize_scores=True)),
    ]
    table = {}
    for name, kw in variants:
        cache = create_kv_cache(name, KVCacheParams(B, Hkv, T, D, Hq), max_chunk_size=q_len, device=dev, **kw)
        # prime: all T rows through the write kernel (it quantises and fills v_norm / q_errors), then the
        # bookkeeping of a cache that has been full for a while
        cache.batch_size, cache.current_length, cache.prefill_length = B, T, T
        idx = torch.arange(T, dtype=torch.int32, device=dev).view(1, 1, T).expand(B, Hkv, T).contiguous()
        cache._write(idx, k, v, 0)
        cache.scores.copy_(torch.rand((B, Hkv, T), device=dev))
        cache._input_pos = T
        cache._use_initial_rule = False
        cache.next_grace_pos = T - cache.grace_period if cache.grace_period else None
        cache.set_next_positions(torch.arange(q_len, dtype=torch.int32, device=dev).view(1, 1, q_len).expand(B, Hkv, q_len))
        for _ in range(max(args.warmup, 2)):
            cache.forward(q, kn, vn)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            cache.forward(q, kn, vn)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.steps
        # cheap invariants of the final state
        tp = cache.token_positions()
        assert int(tp.max()) == cache.input_pos - 1
        if cache.grace_period:
            last = cache.input_pos - 1
            ring = tp[0, 0, T - cache.grace_period:].sort().values.cpu()
            assert torch.equal(ring, torch.arange(last - cache.grace_period + 1, last + 1, dtype=ring.dtype)), "ring lost a recent token"
            assert int(cache._next_index.max()) < T - cache.grace_period
        label = name + "".join(f"+{a}={b}" for a, b in kw.items())
        table[label] = round(ms, 4)
        del cache
    heavy = "qh2o-vlen-torch-quantized8+grace_period=256+normalize_scores=True"
    base = table["h2o-default"]
    flops_alg = 4.0 * B * Hq * q_len * T * D
    return {
        "metric": "H2O cache chunk step with eviction-policy variants, tokens/s of the heaviest variant",
        "value": round(q_len / (table[heavy] * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": table[heavy],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE.json configs[1] shapes (B1 Hq32 Hkv8 D128, 32768 slots, 1024-token chunk) through the cache object, per policy",
            "ms_per_chunk_step": table,
            "overhead_vs_plain_h2o_ms": {kk: round(vv - base, 4) for kk, vv in table.items()},
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "whole chunk step of the heaviest variant (attention + score-sum dominate)",
            "achieved": round(flops_alg / (table[heavy] * 1e-3) / 1e12, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(flops_alg / (table[heavy] * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
            "traffic": None,
        },
        "cpu_baseline": None,
    }


def bench_calib(args, torch, dev):
    n = 1 << 29  # bf16 elements: 1 GiB in, 1 GiB out
    src = torch.ones(n, dtype=torch.bfloat16, device=dev)
    dst = torch.empty_like(src)
    for _ in range(args.warmup):
        torch.neg(src, out=dst)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        torch.neg(src, out=dst)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / args.steps
    return {"metric": "calibration copy GB/s", "value": round(2 * n * 2 / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "elementwise negate, 1 GiB read + 1 GiB written per launch", "bytes_read": 2 * n, "bytes_written": 2 * n}}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path would shard over KV heads without communication; "
              "no multi-GPU code exists). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py: no ROCm device visible; the kernels have no CPU fallback", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    fns = {"prefill": bench_prefill, "quantize": bench_quantize, "decode": bench_decode, "longctx": bench_longctx, "policy": bench_policy, "calib": bench_calib}
    res = fns[args.workload](args, torch, dev)
    if args.workload == "prefill" and args.kv == "bf16" and not args.no_secondary:
        # The other kernels with a target of their own, each on its own configuration, in the same run: the
        # headline fields above stay what they are, these go under config.secondary.
        import copy
        import gc

        secondary = {}
        legs = (("decode", "decode", "bf16", 20, 5), ("quantize", "quantize", "bf16", 20, 5),
                ("prefill_uint8", "prefill", "uint8", 10, 3), ("longctx", "longctx", "bf16", 1, 1))
        for name, workload, kv, steps, warmup in legs:
            sub = copy.copy(args)
            sub.workload, sub.kv, sub.steps, sub.warmup = workload, kv, steps, warmup
            gc.collect()
            torch.cuda.empty_cache()
            t0 = time.perf_counter()
            try:
                r = fns[workload](sub, torch, dev)
                secondary[name] = {"metric": r["metric"], "value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                                   "steps": r["steps"], "warmup": r["warmup"], "dtype": r["dtype"], "workload": r["config"]["workload"],
                                   "detail": {k: v for k, v in r["config"].items() if k != "workload"},
                                   "roofline": r["roofline"], "cpu_baseline": r["cpu_baseline"],
                                   "wall_s": round(time.perf_counter() - t0, 1)}
            except Exception as ex:  # a failing secondary leg must not take the headline measurement with it
                secondary[name] = {"error": f"{type(ex).__name__}: {ex}"}
        res["config"]["secondary"] = secondary
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
