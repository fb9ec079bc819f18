"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and rejects bad requests before touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

from gca_hip import _lib  # noqa: E402


def _header_functions():
    text = open(os.path.join(ROOT, "include", "gca_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:const\s+char\s*\*|int|size_t)\s+(\w+)\s*\(", text, flags=re.M)))


def test_library_exports_every_declared_symbol():
    names = _header_functions()
    assert len(names) >= 11, names
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/gca_hip.h but not exported"
    assert sorted(_lib.SYMBOLS) == names


def test_struct_layout_matches_header():
    # offsets implied by the C declaration order with natural alignment
    assert ctypes.sizeof(_lib.GcaDesc) == 72 and _lib.GcaDesc.Z.offset == 8 and _lib.GcaDesc.N.offset == 56
    assert ctypes.sizeof(_lib.LmkDesc) == 48 and _lib.LmkDesc.E.offset == 24 and _lib.LmkDesc.hidden_size.offset == 40


def _desc(**kw):
    base = dict(dtype=1, w_dtype=0, Z=2, Hq=4, Hkv=2, K=2, Q_CTX=64, K_CTX=64, D=64, sm_scale=0.125, sm_n=0.0,
                path=0, stages=0, N=0, C=0)
    base.update(kw)
    return _lib.GcaDesc(**base)


def test_validation_without_gpu():
    L = _lib.lib()
    assert L.gca_version() >= 100
    one = ctypes.c_void_p(16)   # never dereferenced: validation fails first
    null = ctypes.c_void_p(0)
    assert L.gca_fwd(None, one, one, one, one, one, null, null) == 1
    d = _desc()
    assert L.gca_fwd(ctypes.byref(d), null, one, one, one, one, null, null) == 1
    for bad in (dict(D=48), dict(Hq=3), dict(Z=0), dict(K=0), dict(dtype=7), dict(sm_n=-1.0), dict(path=9)):
        d = _desc(**bad)
        rc = L.gca_fwd(ctypes.byref(d), one, one, one, one, one, null, null)
        assert rc in (2, 3), (bad, rc)
    d = _desc()
    assert L.gca_bwd_workspace_bytes(ctypes.byref(d)) == 2 * 4 * 2 * 64 * 4
    assert L.gca_bwd(ctypes.byref(d), one, one, one, one, one, one, one, one, one, one, null, 0, null) == 5
    d = _desc(N=3, C=4)   # Z % N != 0
    assert L.gca_fwd_indexed(ctypes.byref(d), one, one, one, one, one, one, null, null) == 2
    ld = _lib.LmkDesc(dtype=0, topk=8, N=1, C=4, E=2, Dm=8, causal=1, hidden_size=8.0, reserved=0)
    assert L.lmk_score(ctypes.byref(ld), one, one, one, null) == 2          # causal needs C <= E
    ld = _lib.LmkDesc(dtype=0, topk=8, N=1, C=1, E=1 << 20, Dm=8, causal=1, hidden_size=8.0, reserved=0)
    assert L.lmk_topk_workspace_bytes(ctypes.byref(ld)) > 0
    assert L.lmk_topk(ctypes.byref(ld), one, null, one, one, null, 0, null) == 5
    assert b"workspace" in L.gca_strerror(5)


def test_python_layer_fails_loudly_without_gpu_tensors():
    import torch
    from gca_hip import attention
    q = torch.zeros(1, 1, 64, 64)
    k = torch.zeros(1, 1, 1, 64, 64)
    w = torch.ones(1, 1)
    with pytest.raises(AssertionError):
        attention(q, k, k, w, 0.125, 0.0)


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libgca_hip.so")
    with pytest.raises(RuntimeError):
        _lib.lib()
