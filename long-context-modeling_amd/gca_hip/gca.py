"""Grouped Cross-Attention on MI355X: host side of the HIP kernels.

Mirrors the public surface of the reference's ``ltriton/gca.py``:

* ``attention(q, k, v, weights, sm_scale, sm_n)``   autograd-aware (reference ltriton/gca.py:844,
  class ``_attention`` :681-841); gradients ``(dq, dk, dv, dw, None, None)``.
* ``gca_kv_cache(q, k, v, weights, sm_scale, sm_n)`` inference, any Q_CTX >= 1 (reference :846-888).

and adds the cache-indexed form that skips the K-times-larger gather copies of
model/DRT.py:193-200 and :320-332:

* ``attention_indexed(q, k_cache, v_cache, indices, weights, sm_scale, sm_n)``.

Shapes: q (Z, Hq, Q_CTX, d); k, v (Z, Hkv, K, K_CTX, d); weights (Z, K) shared by all heads
(reference :118); output (Z, Hq, Q_CTX, d) in q's dtype.  k_cache, v_cache (N, C, K_CTX, Hkv*d),
indices (Z, K) int64 with Z % N == 0.

``sm_n`` here is functional: P = exp(s) / (sm_n + sum exp(s)).
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib

_DT = {torch.float32: _lib.GCA_F32, torch.bfloat16: _lib.GCA_BF16}
_PATHS = {"auto": _lib.GCA_PATH_AUTO, "generic": _lib.GCA_PATH_GENERIC, "mfma": _lib.GCA_PATH_MFMA}
_HEAD_DIMS = {16, 32, 64, 128, 256}

# kernel family used by attention()/gca_kv_cache(): "auto", "generic" or "mfma"
kernel_path = "auto"


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _check_inputs(q, k, v, weights):
    # the reference's own preconditions (ltriton/gca.py:688-699, :710-712)
    assert q.is_cuda and k.is_cuda and v.is_cuda and weights.is_cuda, "GCA runs on the GPU only"
    assert q.is_contiguous()
    assert k.is_contiguous()
    assert q.dim() == 4 and k.dim() == 5 and v.shape == k.shape
    assert q.shape[-1] == k.shape[-1] == v.shape[-1]
    assert k.shape[-1] in _HEAD_DIMS, f'current head dim: {k.shape[-1]}'
    assert len(weights.shape) == 2
    assert q.shape[1] % k.shape[1] == 0
    assert q.shape[0] == k.shape[0] == weights.shape[0] and weights.shape[1] == k.shape[2]
    assert q.dtype in _DT, f"unsupported dtype {q.dtype}"
    assert k.dtype == q.dtype and v.dtype == q.dtype
    assert weights.dtype in _DT, f"unsupported weights dtype {weights.dtype}"


def _desc(q, K, K_CTX, Hkv, weights, sm_scale, sm_n, path=None, N=0, C=0):
    Z, Hq, Q_CTX, D = q.shape
    return _lib.GcaDesc(
        dtype=_DT[q.dtype], w_dtype=_DT[weights.dtype], Z=Z, Hq=Hq, Hkv=Hkv, K=K, Q_CTX=Q_CTX, K_CTX=K_CTX, D=D,
        sm_scale=float(sm_scale), sm_n=float(sm_n), path=_PATHS[path or kernel_path], stages=0, N=N, C=C)


def _forward(q, k, v, weights, sm_scale, sm_n, want_lse, path=None):
    _check_inputs(q, k, v, weights)
    v = v.contiguous()
    weights = weights.contiguous()
    Z, Hq, Q_CTX, D = q.shape
    Hkv, K, K_CTX = k.shape[1], k.shape[2], k.shape[3]
    o = torch.empty_like(q)
    lse = torch.empty((Z, Hq, K, Q_CTX), device=q.device, dtype=torch.float32) if want_lse else None
    desc = _desc(q, K, K_CTX, Hkv, weights, sm_scale, sm_n, path)
    with torch.cuda.device(q.device):
        rc = _lib.lib().gca_fwd(ctypes.byref(desc), _ptr(q), _ptr(k), _ptr(v), _ptr(weights), _ptr(o), _ptr(lse),
                                _stream(q.device))
    _lib.check(rc, "gca_fwd")
    return o, lse, v, weights


class _Attention(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, weights, sm_scale, sm_n):
        o, lse, v, weights_c = _forward(q, k, v, weights, sm_scale, sm_n, want_lse=True)
        ctx.save_for_backward(q, k, v, weights_c, lse)
        ctx.sm_scale, ctx.sm_n = float(sm_scale), float(sm_n)
        ctx.w_dtype = weights.dtype
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, weights, lse = ctx.saved_tensors
        do = do.contiguous()
        assert do.shape == q.shape and do.dtype == q.dtype
        Hkv, K, K_CTX = k.shape[1], k.shape[2], k.shape[3]
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dw = torch.empty(weights.shape, device=q.device, dtype=torch.float32)
        desc = _desc(q, K, K_CTX, Hkv, weights, ctx.sm_scale, ctx.sm_n)
        with torch.cuda.device(q.device):
            L = _lib.lib()
            nbytes = L.gca_bwd_workspace_bytes(ctypes.byref(desc))
            ws = torch.empty(nbytes // 4, device=q.device, dtype=torch.float32)
            rc = L.gca_bwd(ctypes.byref(desc), _ptr(q), _ptr(k), _ptr(v), _ptr(weights), _ptr(do), _ptr(lse),
                           _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dw), _ptr(ws), nbytes, _stream(q.device))
        _lib.check(rc, "gca_bwd")
        return dq, dk, dv, dw.to(ctx.w_dtype), None, None


def attention(q, k, v, weights, sm_scale, sm_n=0.0):
    """Training forward with autograd (drop-in for the reference's ``attention``)."""
    return _Attention.apply(q, k, v, weights, sm_scale, sm_n)


def gca_kv_cache(q, k, v, weights, sm_scale, sm_n=0.0):
    """Inference forward: no autograd, nothing saved, any Q_CTX >= 1."""
    with torch.no_grad():
        return _forward(q, k, v, weights, sm_scale, sm_n, want_lse=False)[0]


# ------------------------------------------------------------------------------- indexed form

def _check_indexed(q, k_cache, v_cache, indices, weights):
    assert q.is_cuda and q.is_contiguous() and q.dim() == 4
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape and k_cache.dim() == 4
    assert q.dtype in _DT and k_cache.dtype == q.dtype and v_cache.dtype == q.dtype
    assert indices.dtype == torch.int64 and indices.is_contiguous() and indices.shape == weights.shape
    assert weights.dim() == 2 and weights.shape[0] == q.shape[0] and weights.dtype in _DT
    Z, Hq, _, D = q.shape
    N, C, K_CTX, Dm = k_cache.shape
    assert D in _HEAD_DIMS, f'current head dim: {D}'
    assert Dm % D == 0 and Hq % (Dm // D) == 0 and Z % N == 0
    return N, C, K_CTX, Dm // D


class _AttentionIndexed(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k_cache, v_cache, indices, weights, sm_scale, sm_n):
        N, C, K_CTX, Hkv = _check_indexed(q, k_cache, v_cache, indices, weights)
        weights_c = weights.contiguous()
        Z, Hq, Q_CTX, D = q.shape
        K = indices.shape[1]
        o = torch.empty_like(q)
        lse = torch.empty((Z, Hq, K, Q_CTX), device=q.device, dtype=torch.float32)
        desc = _desc(q, K, K_CTX, Hkv, weights_c, sm_scale, sm_n, N=N, C=C)
        with torch.cuda.device(q.device):
            rc = _lib.lib().gca_fwd_indexed(ctypes.byref(desc), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(indices),
                                            _ptr(weights_c), _ptr(o), _ptr(lse), _stream(q.device))
        _lib.check(rc, "gca_fwd_indexed")
        ctx.save_for_backward(q, k_cache, v_cache, indices, weights_c, lse)
        ctx.sm_scale, ctx.sm_n, ctx.w_dtype = float(sm_scale), float(sm_n), weights.dtype
        return o

    @staticmethod
    def backward(ctx, do):
        q, k_cache, v_cache, indices, weights, lse = ctx.saved_tensors
        do = do.contiguous()
        N, C, K_CTX, Dm = k_cache.shape
        Hkv, K = Dm // q.shape[-1], indices.shape[1]
        dq = torch.empty_like(q)
        dkc, dvc = torch.empty_like(k_cache), torch.empty_like(v_cache)
        dw = torch.empty(weights.shape, device=q.device, dtype=torch.float32)
        desc = _desc(q, K, K_CTX, Hkv, weights, ctx.sm_scale, ctx.sm_n, N=N, C=C)
        with torch.cuda.device(q.device):
            L = _lib.lib()
            nbytes = L.gca_bwd_workspace_bytes(ctypes.byref(desc))
            ws = torch.empty(nbytes // 4, device=q.device, dtype=torch.float32)
            rc = L.gca_bwd_indexed(ctypes.byref(desc), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(indices),
                                   _ptr(weights), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dkc), _ptr(dvc), _ptr(dw),
                                   _ptr(ws), nbytes, _stream(q.device))
        _lib.check(rc, "gca_bwd_indexed")
        return dq, dkc, dvc, None, dw.to(ctx.w_dtype), None, None


def attention_indexed(q, k_cache, v_cache, indices, weights, sm_scale, sm_n=0.0):
    """GCA reading retrieved chunks from the chunk cache by index (autograd-aware).

    Equals ``attention(q, gather(k_cache), gather(v_cache), weights, ...)`` where the gather is
    ``cache[n, indices]`` rearranged to (Z, Hkv, K, K_CTX, d); gradients of the caches are summed
    over all query chunks that retrieved a chunk.
    """
    return _AttentionIndexed.apply(q, k_cache, v_cache, indices, weights, sm_scale, sm_n)


def gca_kv_cache_indexed(q, k_cache, v_cache, indices, weights, sm_scale, sm_n=0.0):
    """Inference form of ``attention_indexed`` (no autograd, no LSE written)."""
    with torch.no_grad():
        N, C, K_CTX, Hkv = _check_indexed(q, k_cache, v_cache, indices, weights)
        weights = weights.contiguous()
        o = torch.empty_like(q)
        desc = _desc(q, indices.shape[1], K_CTX, Hkv, weights, sm_scale, sm_n, N=N, C=C)
        with torch.cuda.device(q.device):
            rc = _lib.lib().gca_fwd_indexed(ctypes.byref(desc), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(indices),
                                            _ptr(weights), _ptr(o), ctypes.c_void_p(0), _stream(q.device))
        _lib.check(rc, "gca_fwd_indexed")
        return o
