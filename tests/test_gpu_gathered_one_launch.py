"""Gathered-form backward in one launch (bf16, d = 64, 1 / 2 / 4 query heads per kv head, 64 query rows): dq, dk and
dv from the same pass over K / V.

Checked against the oracle like every other path, and against the staged form of the same entry point
(``desc.stages`` = dq alone, then dk/dv alone, which runs the two separate kernels): both round P and dS to bf16 once
and accumulate in fp32 (the separate dk/dv kernel on pre-scaled operands), so they agree to bf16 output rounding.  Weights include zeros (the slot's dk / dv must
be written as zeros), negatives, and bf16 storage.
"""
import ctypes

import pytest
import torch

from helpers import gca_inputs, oracle64, rel_err

pytestmark = pytest.mark.gpu

DQ, DKDV, DW = 1, 2, 4


def _bwd(q, k, v, w, do, lse, sm_scale, stages_seq):
    from gca_hip import _lib
    from gca_hip.gca import _desc, _ptr, _stream
    Hkv, K, K_CTX = k.shape[1], k.shape[2], k.shape[3]
    dq, dk, dv = torch.full_like(q, float("nan")), torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
    dw = torch.full(w.shape, float("nan"), device=q.device, dtype=torch.float32)
    desc = _desc(q, K, K_CTX, Hkv, w, sm_scale, 0.0, "mfma")
    L = _lib.lib()
    nbytes = L.gca_bwd_workspace_bytes(ctypes.byref(desc))
    ws = torch.empty(nbytes // 4, device=q.device, dtype=torch.float32)
    for stages in stages_seq:
        desc.stages = stages
        rc = L.gca_bwd(ctypes.byref(desc), _ptr(q), _ptr(k), _ptr(v), _ptr(w), _ptr(do), _ptr(lse), _ptr(dq), _ptr(dk),
                       _ptr(dv), _ptr(dw), _ptr(ws), nbytes, _stream(q.device))
        _lib.check(rc, "gca_bwd")
    torch.cuda.synchronize()
    return dq, dk, dv, dw


@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Z,Hq,Hkv,K", [(3, 2, 2, 1), (5, 3, 3, 3), (7, 12, 12, 8), (2, 1, 1, 16), (64, 4, 4, 5),
                                        (5, 4, 2, 3), (4, 2, 1, 5), (9, 6, 3, 8),          # two query heads per kv head
                                        (3, 8, 2, 4), (6, 4, 1, 8), (17, 12, 3, 2)])       # four
def test_one_launch_equals_staged_form_and_oracle(Z, Hq, Hkv, K, w_dtype):
    from gca_hip.gca import _forward
    S, d = 64, 64
    q, k, v, w, do = gca_inputs(Z, Hq, Hkv, K, S, S, d, torch.bfloat16, seed=900 + Z + K, w_dtype=torch.float32)
    g = torch.Generator().manual_seed(901 + K)
    w = torch.randn(Z, K, generator=g)
    if K > 1:
        w[:, 1] = 0.0                                    # a dead slot in every row
    w[0] = -w[0].abs()                                   # a row of negative weights only
    w = w.to(w_dtype)
    ref = oracle64(q, k, v, w.float(), do, d ** -0.5, 0.0)
    qd, kd, vd, wd, dod = [t.cuda() for t in (q, k, v, w, do)]
    o, lse, _, _ = _forward(qd, kd, vd, wd, d ** -0.5, 0.0, want_lse=True, path="mfma")
    one = _bwd(qd, kd, vd, wd, dod, lse, d ** -0.5, [0])                  # all stages: the one-launch kernel
    two = _bwd(qd, kd, vd, wd, dod, lse, d ** -0.5, [DQ, DKDV, DW])       # the separate dq and dk/dv kernels
    for name, a, b, r in zip("dq dk dv dw".split(), one, two, ref[1:]):
        assert torch.isfinite(a.float()).all(), name                      # every element written
        assert rel_err(a, r) <= 2e-2, (name, rel_err(a, r))
        assert rel_err(a, b.float().cpu()) <= 1.5e-2, (name, rel_err(a, b.float().cpu()))
    if K > 1:
        assert (one[1][:, :, 1] == 0).all() and (one[2][:, :, 1] == 0).all()

