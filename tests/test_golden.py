"""Golden fixtures: the oracle must keep reproducing them (CPU), and the HIP path must match
them (GPU).  tests/golden/make_golden.py documents how they were made."""
import importlib.util
import json
import os

import numpy as np
import pytest
import torch

from oracle import gca_oracle as orc

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "make_golden.py"))
mk = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(mk)


def _tiny():
    z = np.load(os.path.join(HERE, "gca_tiny_fp32.npz"))
    return {k: torch.from_numpy(z[k]) for k in z.files}


def _digest_of(t):
    t = t.detach().double().cpu()
    return {"sum": float(t.sum()), "abs_sum": float(t.abs().sum()), "max_abs": float(t.abs().max()),
            "head": [float(x) for x in t.flatten()[:8]], "stride_sample": [float(x) for x in t.flatten()[::100003][:16]]}


def _close(a, b, rtol, scale):
    return abs(a - b) <= rtol * max(scale, abs(b))


def _check_digest(got, ref, rtol):
    scale = ref["max_abs"]
    n = 1.0
    assert _close(got["max_abs"], ref["max_abs"], rtol, scale)
    assert _close(got["abs_sum"], ref["abs_sum"], rtol, ref["abs_sum"])
    for a, b in zip(got["head"] + got["stride_sample"], ref["head"] + ref["stride_sample"]):
        assert _close(a, b, rtol, scale), (a, b)


def test_lcg_inputs_are_reproducible():
    t = _tiny()
    assert torch.equal(mk.lcg_normal(tuple(t["q_all"].shape), 7, 0.5), t["q_all"])
    x = mk.lcg_normal((100000,), 3)
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 1.0) < 0.02


def test_oracle_reproduces_tiny_fixture():
    t = _tiny()
    a = [t[k].double().requires_grad_(True) for k in ("q_all", "chunk_k", "chunk_v")]
    out, idx, w = orc.gca_layer(a[0], a[1], a[2], t["lmk_q"].double(), t["lmk_k"].double(), 3, 2, sm_n=1.0)
    out.backward(t["dout"].double())
    assert torch.equal(idx, t["indices"])
    assert torch.allclose(w, t["weights"], atol=1e-12)
    for got, name in ((out, "out"), (a[0].grad, "dq"), (a[1].grad, "dk"), (a[2].grad, "dv")):
        assert torch.allclose(got, t[name], rtol=1e-10, atol=1e-12), name


def test_oracle_reproduces_cfg1_digest():
    ref = json.load(open(os.path.join(HERE, "gca_cfg1_digest.json")))
    r = ref["recipe"]
    c = mk.layer_case(r["N"], r["C"], r["Hq"], r["Hkv"], r["S"], r["d"], r["K"], r["sm_n"], r["seed"])
    assert c["indices"].tolist() == ref["indices"]
    for name in ("out", "dq", "dk", "dv"):
        _check_digest(_digest_of(c[name]), ref[name], 1e-9)


@pytest.mark.gpu
def test_hip_matches_tiny_fixture():
    import gca_hip
    t = _tiny()
    dev = "cuda"
    a = [t[k].to(dev).requires_grad_(True) for k in ("q_all", "chunk_k", "chunk_v")]
    out, idx, w = gca_hip.gca_layer(a[0], a[1], a[2], t["lmk_q"].to(dev), t["lmk_k"].to(dev), 3, sm_n=1.0)
    out.backward(t["dout"].to(dev))
    assert torch.equal(idx.cpu(), t["indices"])
    assert (w.cpu().double() - t["weights"]).abs().max() <= 1e-6
    for got, name in ((out, "out"), (a[0].grad, "dq"), (a[1].grad, "dk"), (a[2].grad, "dv")):
        ref = t[name]
        err = (got.detach().double().cpu() - ref).abs().max().item() / ref.abs().max().item()
        assert err <= 1e-5, f"{name}: {err:.2e}"


@pytest.mark.gpu
def test_hip_matches_cfg1_digest():
    import gca_hip
    ref = json.load(open(os.path.join(HERE, "gca_cfg1_digest.json")))
    r = ref["recipe"]
    dev = "cuda"
    q_all = mk.lcg_normal((r["N"], r["C"], r["Hq"], r["S"], r["d"]), r["seed"], 0.5).to(dev).requires_grad_(True)
    ck = mk.lcg_normal((r["N"], r["C"], r["S"], r["Hkv"] * r["d"]), r["seed"] + 1, 0.5).to(dev).requires_grad_(True)
    cv = mk.lcg_normal((r["N"], r["C"], r["S"], r["Hkv"] * r["d"]), r["seed"] + 2, 0.5).to(dev).requires_grad_(True)
    lq = mk.lcg_normal((r["N"], r["C"], r["Hkv"] * r["d"]), r["seed"] + 3).to(dev)
    lk = mk.lcg_normal((r["N"], r["C"], r["Hkv"] * r["d"]), r["seed"] + 4).to(dev)
    do = mk.lcg_normal((r["N"], r["C"], r["Hq"], r["S"], r["d"]), r["seed"] + 5).to(dev)
    out, idx, w = gca_hip.gca_layer(q_all, ck, cv, lq, lk, r["K"], sm_n=r["sm_n"])
    out.backward(do)
    assert idx.cpu().tolist() == ref["indices"]
    assert (w.cpu().double() - torch.tensor(ref["weights"], dtype=torch.float64)).abs().max() <= 1e-6
    for got, name in ((out, "out"), (q_all.grad, "dq"), (ck.grad, "dk"), (cv.grad, "dv")):
        _check_digest(_digest_of(got), ref[name], 1e-5)
