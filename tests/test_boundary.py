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
    assert kvx.kvx_version() == 101


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
    a.D = 256
    assert kvx.kvx_sdpa_prefill(ctypes.byref(a), None) == _lib.KVX_ERR_UNSUPPORTED
    h = _lib.H2OArgs()
    h.B, h.Hkv, h.kv_len, h.limit, h.k = 1, 1, 16, 16, 17
    assert kvx.kvx_h2o_update_select(ctypes.byref(h), None) == _lib.KVX_ERR_INVALID
    assert kvx.kvx_device_count() >= 0


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
    with pytest.raises(NotImplementedError):
        s.scaled_dot_product_attention(q.half(), k.half(), k.half(), None, 6, None)
    with pytest.raises(NotImplementedError, match="q_len=1, kv_len=1"):
        s.scaled_dot_product_attention(q[:, :, :1], k[:, :, :1], k[:, :, :1], None, 6, None)


def test_c_oracle_builds():
    from oracle import c_oracle

    assert os.path.exists(c_oracle.build())
