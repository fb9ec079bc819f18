"""lmk_score_topk_static: the retrieval entry point that allocates nothing (scores and top-k scratch live in a
static device array inside the library).  Called through the C ABI and compared with lmk_score_topk, which takes
caller-allocated buffers: indices must be identical and the weights bit-equal, on two calls in a row of which the
second is smaller (the shared scratch still holds the first call's data), for the decode shapes of BASELINE
config 5 and a training-shaped block with noise."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(lq, lk, topk, causal=True, noise=None):
    from gca_hip import _lib
    from gca_hip.gca import _ptr, _stream
    from gca_hip.retrieval import _lmk_desc
    L = _lib.lib()
    N, C, Dm = lq.shape
    E = lk.shape[1]
    kk = min(E, topk)
    desc = _lmk_desc(lq.dtype, topk, N, C, E, Dm, causal, Dm)
    stream = _stream(lq.device)
    # existing entry point: caller-allocated scores and workspace
    scores = torch.empty((N, C, E), device=DEV, dtype=lq.dtype)
    nws = L.lmk_topk_workspace_bytes(ctypes.byref(desc))
    ws = torch.empty(max(nws, 8) // 8, device=DEV, dtype=torch.int64)
    idx_a = torch.empty((N, C, kk), device=DEV, dtype=torch.int64)
    w_a = torch.empty((N, C, kk), device=DEV, dtype=torch.float32)
    _lib.check(L.lmk_score_topk(ctypes.byref(desc), _ptr(lq), _ptr(lk), _ptr(noise), _ptr(scores), _ptr(idx_a), _ptr(w_a),
                                _ptr(ws), nws, stream), "lmk_score_topk")
    # the entry point under test: inputs and outputs only
    idx_b = torch.full((N, C, kk), -7, device=DEV, dtype=torch.int64)
    w_b = torch.full((N, C, kk), -7.0, device=DEV, dtype=torch.float32)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = L.lmk_score_topk_static(ctypes.byref(desc), _ptr(lq), _ptr(lk), _ptr(noise), _ptr(idx_b), _ptr(w_b), stream)
    _lib.check(rc, "lmk_score_topk_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return (idx_a, w_a), (idx_b, w_b)


def _rand(shape, seed, dtype):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn(*shape, device=DEV, generator=g).to(dtype)


def test_static_entry_point_equals_lmk_score_topk_two_calls_in_a_row():
    Dm, K = 768, 8
    # first call: one decode row against 262144 cached landmarks (bf16: 0.5 MiB of scores, segmented top-k)
    lq, lk = _rand((1, 1, Dm), 1, torch.bfloat16), _rand((1, 262144, Dm), 2, torch.bfloat16)
    (ia, wa), (ib, wb) = _both(lq, lk, K)
    assert torch.equal(ia, ib) and torch.equal(wa, wb)
    assert (wb.sum(-1) - 1).abs().max() <= 1e-5
    # second call, smaller, on the same GPU right after it: 64 sequences x 1024 landmarks
    lq, lk = _rand((64, 1, Dm), 3, torch.bfloat16), _rand((64, 1024, Dm), 4, torch.bfloat16)
    (ia, wa), (ib, wb) = _both(lq, lk, K)
    assert torch.equal(ia, ib) and torch.equal(wa, wb)
    # third, smaller again: fp32 training-shaped block with selection noise, rows that see fewer than k chunks
    lq, lk = _rand((2, 40, 64), 5, torch.float32), _rand((2, 40, 64), 6, torch.float32)
    noise = _rand((2, 40, 40), 7, torch.float32)
    (ia, wa), (ib, wb) = _both(lq, lk, 4, True, noise)
    assert torch.equal(ia, ib) and torch.equal(wa, wb)
    assert (wb[:, 0] == 0).all()


def test_python_wrapper_writes_into_caller_tensors():
    import gca_hip
    lq, lk = _rand((4, 1, 256), 10, torch.bfloat16), _rand((4, 900, 256), 11, torch.bfloat16)
    _, idx, w = gca_hip.landmark_retrieve(lq, lk, 8, 256)
    oi = torch.empty((4, 1, 8), device=DEV, dtype=torch.int64)
    ow = torch.empty((4, 1, 8), device=DEV, dtype=torch.float32)
    gca_hip.landmark_retrieve_static(lq, lk, 8, oi, ow, 256)
    assert torch.equal(oi, idx) and torch.equal(ow, w)


def test_static_entry_point_rejects_what_does_not_fit():
    from gca_hip import _lib
    from gca_hip.gca import _ptr, _stream
    from gca_hip.retrieval import _lmk_desc
    L = _lib.lib()
    # 4096 x 4096 fp32 scores = 64 MiB > 8 MiB: refused before anything is launched, outputs untouched
    N, C, Dm = 1, 4096, 64
    lq, lk = _rand((N, C, Dm), 8, torch.float32), _rand((N, C, Dm), 9, torch.float32)
    idx = torch.full((N, C, 8), -7, device=DEV, dtype=torch.int64)
    w = torch.full((N, C, 8), -7.0, device=DEV, dtype=torch.float32)
    desc = _lmk_desc(lq.dtype, 8, N, C, C, Dm, True, Dm)
    rc = L.lmk_score_topk_static(ctypes.byref(desc), _ptr(lq), _ptr(lk), _ptr(None), _ptr(idx), _ptr(w), _stream(lq.device))
    assert rc == _lib.GCA_ERR_SCRATCH_LIMIT
    assert b"static scratch" in L.gca_strerror(rc)
    torch.cuda.synchronize()
    assert (idx == -7).all() and (w == -7.0).all()
    # sizes whose product overflows 64 bits are refused the same way
    desc = _lmk_desc(lq.dtype, 8, 1 << 40, 1 << 40, 1 << 30, Dm, False, Dm)
    assert L.lmk_score_topk_static(ctypes.byref(desc), _ptr(lq), _ptr(lk), _ptr(None), _ptr(idx), _ptr(w),
                                   _stream(lq.device)) == _lib.GCA_ERR_SCRATCH_LIMIT
