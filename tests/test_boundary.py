"""CPU-side checks of the drop-in boundary: the C-ABI library loads, exports every symbol that
include/kvx.h declares, the ctypes structs match the C layout, argument validation answers without
a GPU, and the host classes keep the reference's error behaviour. No kernel is launched here."""
import ctypes
import os
import re
import subprocess
import tempfile

import pytest
import torch

from keys_values_amd import _lib
from keys_values_amd.attention import ops
from keys_values_amd.attention.sdpa import HipSDPA

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "kvx.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(kvx):
    names = _declared_symbols()
    assert len(names) >= 15
    assert sorted(_lib.SYMBOLS) == names, "ctypes table and header disagree"
    for n in names:
        assert hasattr(kvx, n), f"libkvx.so does not export {n}"
    assert kvx.kvx_version() == 103


def test_struct_layouts_match_c(tmp_path):
    src = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void){"]
    structs = {"kvx_sdpa_args": _lib.SdpaArgs, "kvx_cache_write_args": _lib.CacheWriteArgs, "kvx_h2o_args": _lib.H2OArgs}
    for cname, cls in structs.items():
        src.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            src.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    src.append("return 0;}")
    c = tmp_path / "layout.c"
    c.write_text("\n".join(src))
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", str(c), "-o", str(exe)])
    got = dict(line.split() for line in subprocess.check_output([str(exe)], text=True).splitlines())
    for cname, cls in structs.items():
        assert int(got[cname]) == ctypes.sizeof(cls)
        for fname, _ in cls._fields_:
            assert int(got[f"{cname}.{fname}"]) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_validation_answers_without_a_gpu(kvx):
    # argument checks come before any HIP call
    rc = kvx.kvx_quantize_rows(None, 100, 4, 100, None, None, None, None)
    assert rc == _lib.KVX_ERR_UNSUPPORTED and b"row length 100" in kvx.kvx_last_error()
    with pytest.raises(NotImplementedError):
        _lib.check(rc)
    a = _lib.SdpaArgs()
    a.B, a.Hq, a.Hkv, a.q_len, a.kv_len, a.D = 1, 6, 4, 8, 16, 128
    a.sm_scale = 0.1
    rc = kvx.kvx_sdpa_prefill(ctypes.byref(a), None)
    assert rc == _lib.KVX_ERR_INVALID and b"multiple of Hkv" in kvx.kvx_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    a.Hq = 8
    a.D = 512
    assert kvx.kvx_sdpa_prefill(ctypes.byref(a), None) == _lib.KVX_ERR_UNSUPPORTED
    a.D, a.kv_dtype = 128, 17  # not a store type
    assert kvx.kvx_sdpa_prefill(ctypes.byref(a), None) == _lib.KVX_ERR_UNSUPPORTED and b"kv_dtype" in kvx.kvx_last_error()
    a.kv_dtype = _lib.KVX_KV_BF16
    h = _lib.H2OArgs()
    h.B, h.Hkv, h.kv_len, h.limit, h.k = 1, 1, 16, 16, 17
    assert kvx.kvx_h2o_update_select(ctypes.byref(h), None) == _lib.KVX_ERR_INVALID
    assert kvx.kvx_device_count() >= 0


def test_random_arguments_are_answered_not_trusted(kvx):
    """Seeded random argument blocks (sizes from a set of edge values, pointers NULL / aligned /
    misaligned, strides zero / negative / odd) through every entry point that takes one: each call must
    come back with a status (no division by a zero size, no walk over a NULL pointer on the host).
    Only where no device is visible: a block that happens to pass every check would be launched."""
    import random

    if kvx.kvx_device_count() > 0:
        pytest.skip("a device is visible: random pointers must not reach a kernel")
    rnd = random.Random(2024)
    ints = [-1, 0, 1, 2, 3, 7, 8, 64, 100, 128, 256, 4096, 4097, 2**31 - 1]
    ptrs = [0, 0, 0x10000, 0x10008, 0x10001]
    strides = [-8, 0, 1, 8, 64, 128, 1024, 2**40]
    codes = {_lib.KVX_OK, _lib.KVX_ERR_INVALID, _lib.KVX_ERR_UNSUPPORTED, _lib.KVX_ERR_WORKSPACE, _lib.KVX_ERR_HIP}

    def fill(obj):
        for name, ctype in obj._fields_:
            if ctype is ctypes.c_void_p:
                v = rnd.choice(ptrs)
            elif ctype is ctypes.c_int64 or ctype is ctypes.c_size_t:
                v = rnd.choice(strides)
                if ctype is ctypes.c_size_t:
                    v = abs(v)
            elif ctype is ctypes.c_int32:
                v = rnd.choice(ints)
            else:
                v = rnd.choice([-1.0, 0.0, 0.125, 0.5, 2.0])
            setattr(obj, name, v)
        return obj

    def valid_sdpa():
        a = _lib.SdpaArgs()
        a.B, a.Hkv, a.D, a.kv_dtype = rnd.choice([1, 2]), rnd.choice([1, 2]), rnd.choice([64, 128]), rnd.choice([0, 1, 2])
        a.Hq = a.Hkv * rnd.choice([1, 2, 4])
        a.kv_len = rnd.choice([1, 63, 64, 1000, 70000])
        a.q_len = rnd.choice([1, min(a.kv_len, 100)])
        a.input_pos, a.sm_scale = a.kv_len - a.q_len, 0.125
        for name, ctype in a._fields_:
            if ctype is ctypes.c_void_p:
                setattr(a, name, 0x10000)
        a.q_stride_t = a.k_stride_t = a.v_stride_t = a.o_stride_h = a.D
        a.q_stride_h, a.k_stride_h = a.q_len * a.D, a.kv_len * a.D
        a.v_stride_h, a.o_stride_t = a.k_stride_h, a.Hq * a.D
        a.q_stride_b, a.k_stride_b = a.Hq * a.q_stride_h, a.Hkv * a.k_stride_h
        a.v_stride_b, a.o_stride_b = a.k_stride_b, a.q_len * a.o_stride_t
        a.qs_stride_h = a.tp_stride_h = a.kv_len
        a.qs_stride_b = a.tp_stride_b = a.Hkv * a.kv_len
        a.workspace_bytes = 1 << 40
        return a

    def mutate(obj, times):
        for _ in range(times):
            name, ctype = rnd.choice(obj._fields_)
            if ctype is ctypes.c_void_p:
                setattr(obj, name, rnd.choice(ptrs))
            elif ctype is ctypes.c_int64 or ctype is ctypes.c_size_t:
                setattr(obj, name, abs(rnd.choice(strides)) if ctype is ctypes.c_size_t else rnd.choice(strides))
            elif ctype is ctypes.c_int32:
                setattr(obj, name, rnd.choice(ints))
            else:
                setattr(obj, name, rnd.choice([-1.0, 0.0, 0.125, 0.5, 2.0]))
        return obj

    for it in range(600):
        # half of the blocks are random throughout, half are valid ones with up to two fields replaced
        a = fill(_lib.SdpaArgs()) if it % 2 else mutate(valid_sdpa(), rnd.choice([0, 1, 1, 2]))
        h = fill(_lib.H2OArgs())
        for fn in (kvx.kvx_sdpa_prefill, kvx.kvx_score_sum, kvx.kvx_sdpa_decode):
            assert fn(ctypes.byref(a), None) in codes
        assert kvx.kvx_sdpa_decode_h2o(ctypes.byref(a), ctypes.byref(h), None) in codes
        for fn in (kvx.kvx_sdpa_prefill_workspace_bytes, kvx.kvx_sdpa_decode_workspace_bytes, kvx.kvx_sdpa_decode_h2o_workspace_bytes):
            assert fn(ctypes.byref(a)) >= 0
        assert kvx.kvx_h2o_update_select(ctypes.byref(h), None) in codes
        assert kvx.kvx_h2o_workspace_bytes(ctypes.byref(h)) >= 0
        assert kvx.kvx_cache_write(ctypes.byref(fill(_lib.CacheWriteArgs())), None) in codes
        q = fill(_lib.BlockQuantArgs())
        assert kvx.kvx_quantize_blocks(ctypes.byref(q), None) in codes
        assert kvx.kvx_dequantize_blocks(ctypes.byref(q), None) in codes
        r = lambda: rnd.choice(ptrs)  # noqa: E731
        n, d, st = rnd.choice(ints), rnd.choice(ints), rnd.choice(strides)
        assert kvx.kvx_quantize_rows(r(), st, n, d, r(), r(), r(), None) in codes
        assert kvx.kvx_dequantize_rows(r(), r(), r(), n, d, r(), st, None) in codes
        assert kvx.kvx_quantize_rows4(r(), st, n, d, r(), r(), r(), None) in codes
        assert kvx.kvx_dequantize_rows4(r(), r(), r(), n, d, r(), st, None) in codes
        assert kvx.kvx_rmsnorm_rows(r(), st, r(), st, r(), n, d, 1e-6, None) in codes
        assert kvx.kvx_add_rmsnorm_rows(r(), st, r(), st, r(), st, r(), st, r(), n, d, 1e-6, None) in codes
        assert kvx.kvx_swiglu_rows(r(), st, r(), st, n, d, None) in codes
        assert kvx.kvx_qk_norm_rope(r(), st, st, rnd.choice(ints), n, rnd.choice(ints), rnd.choice(ints), d, r(), r(), 1e-6, r(), r(),
                                    rnd.choice(ints), rnd.choice(ints), None) in codes


def test_no_cpu_fallback():
    q = torch.zeros(1, 4, 2, 64, dtype=torch.bfloat16)
    k = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.prefill_core(q, k, k, 0.125, 6)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.decode_core(q[:, :, :1], k, k, 0.125)


def test_load_error_is_reported(monkeypatch, tmp_path):
    # keys_values/attention/flashinfer_ops.py:86-147: a failed load leaves a message, a good one None
    from keys_values_amd import attention

    _lib.load()
    assert attention.get_load_error() is None
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "_load_error", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libkvx.so"))
    with pytest.raises(ImportError):
        _lib.load()
    assert "not found" in attention.get_load_error()
    assert not attention.is_available()
    monkeypatch.undo()
    _lib.load()
    assert attention.get_load_error() is None


def test_hip_sdpa_keeps_reference_errors():
    # keys_values/attention/flashinfer_wrapper.py:406-432, keys_values/attention/sdpa_wrapper.py:24-47
    s = HipSDPA.__new__(HipSDPA)
    q = torch.zeros(1, 4, 2, 64, dtype=torch.bfloat16)
    k = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="input_pos must be positive"):
        s.scaled_dot_product_attention(q, k, k, None, 0, None)
    with pytest.raises(ValueError, match="int scalar"):
        s.scaled_dot_product_attention(q, k, k, None, 1.0, None)
    with pytest.raises(ValueError, match="same shape"):
        s.scaled_dot_product_attention(q, k, k[:, :, :4], None, 6, None)
    with pytest.raises(ValueError, match="q_len"):
        s.scaled_dot_product_attention(torch.zeros(1, 4, 9, 64, dtype=torch.bfloat16), k, k, None, 6, None)
    with pytest.raises(ValueError, match="multiple of n_query_groups"):
        s.scaled_dot_product_attention(torch.zeros(1, 3, 2, 64, dtype=torch.bfloat16), k, k, None, 6, None)
    with pytest.raises(ValueError, match="Not compatible"):
        s.scaled_dot_product_attention(q, k, k, None, 6, torch.zeros(1, 2, 7, dtype=torch.int32))
    with pytest.raises(NotImplementedError):  # float32 is not served (float16 and bfloat16 are, as in the reference)
        s.scaled_dot_product_attention(q.float(), k.float(), k.float(), None, 6, None)
    with pytest.raises(NotImplementedError, match="head_size <= 256"):
        s.scaled_dot_product_attention(torch.zeros(1, 4, 2, 264, dtype=torch.bfloat16), torch.zeros(1, 2, 8, 264, dtype=torch.bfloat16),
                                       torch.zeros(1, 2, 8, 264, dtype=torch.bfloat16), None, 6, None)
    with pytest.raises(NotImplementedError, match="q_len=1, kv_len=1"):
        s.scaled_dot_product_attention(q[:, :, :1], k[:, :, :1], k[:, :, :1], None, 6, None)


def test_bench_refuses_more_than_one_gpu_and_runs_nothing_without_one():
    import sys

    bench = os.path.join(ROOT, "bench.py")
    r = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""
    if not torch.cuda.is_available():  # no device: it must say so, not fall back to the CPU
        r = subprocess.run([sys.executable, bench, "--steps", "1", "--warmup", "0"], capture_output=True, text=True)
        assert r.returncode != 0 and "no CPU fallback" in r.stderr and r.stdout.strip() == ""


def test_c_oracle_builds():
    from oracle import c_oracle

    assert os.path.exists(c_oracle.build())
