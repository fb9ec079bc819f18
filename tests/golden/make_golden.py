#!/usr/bin/env python3
"""Writes the golden fixtures of this directory with the CPU oracle (float64).

The reference keeps no vectors for this path (its kernel test draws inputs from the GPU RNG,
ltriton/gca.py:895-908), so these are produced by the oracle, whose formulas are pinned
independently in tests/test_oracle.py.  They guard the oracle against drift and give the HIP
path fixed inputs/outputs that do not depend on any RNG implementation.

  gca_tiny_fp32.npz   every input and output of one small GCA layer (fp32 inputs):
                      N=2, C=5, Hq=4, Hkv=2, S=16, d=16, top-k 3, softmax-off-by-one on
  gca_cfg1_digest.json  BASELINE config 1 (B=2, H=4, d=64, L=1024, chunk 64, top-k 4, fp32):
                      inputs are regenerated from the integer recipe below; the file holds the
                      retrieval indices and slices / sums of the outputs and gradients

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import gca_oracle as orc  # noqa: E402


def lcg_normal(shape, seed, scale=1.0):
    """Deterministic pseudo-normal floats from integer arithmetic only (sum of 4 LCG uniforms),
    so the same inputs can be rebuilt anywhere without relying on a library RNG."""
    n = int(np.prod(shape))
    idx = np.arange(n * 4, dtype=np.uint64) + np.uint64(seed) * np.uint64(1_000_003)
    x = idx * np.uint64(6364136223846793005) + np.uint64(1442695040888963407)
    x ^= x >> np.uint64(33)
    x *= np.uint64(0xff51afd7ed558ccd)
    x ^= x >> np.uint64(33)
    u = (x >> np.uint64(40)).astype(np.float64) / float(1 << 24)          # [0, 1)
    z = (u.reshape(n, 4).sum(1) - 2.0) * np.sqrt(3.0)                      # mean 0, var 1
    return torch.from_numpy((z * scale).astype(np.float32).reshape(shape))


def layer_case(N, C, Hq, Hkv, S, d, K, sm_n, seed):
    q_all = lcg_normal((N, C, Hq, S, d), seed, 0.5)
    ck = lcg_normal((N, C, S, Hkv * d), seed + 1, 0.5)
    cv = lcg_normal((N, C, S, Hkv * d), seed + 2, 0.5)
    lq = lcg_normal((N, C, Hkv * d), seed + 3)
    lk = lcg_normal((N, C, Hkv * d), seed + 4)
    do = lcg_normal((N, C, Hq, S, d), seed + 5)
    a = [t.double().requires_grad_(True) for t in (q_all, ck, cv)]
    out, idx, w = orc.gca_layer(a[0], a[1], a[2], lq.double(), lk.double(), K, Hkv, sm_n=sm_n)
    out.backward(do.double())
    scores = orc.mask_scores(orc.landmark_scores(lq.double(), lk.double()))
    return dict(q_all=q_all, chunk_k=ck, chunk_v=cv, lmk_q=lq, lmk_k=lk, dout=do, scores=scores, indices=idx,
                weights=w, out=out.detach(), dq=a[0].grad, dk=a[1].grad, dv=a[2].grad)


def main():
    tiny = layer_case(2, 5, 4, 2, 16, 16, 3, 1.0, seed=7)
    np.savez_compressed(os.path.join(HERE, "gca_tiny_fp32.npz"),
                        **{k: (v.numpy() if v.dtype != torch.float64 else v.numpy().astype(np.float64))
                           for k, v in tiny.items()})
    c1 = layer_case(2, 16, 4, 4, 64, 64, 4, 1.0, seed=11)
    digest = {"recipe": dict(N=2, C=16, Hq=4, Hkv=4, S=64, d=64, K=4, sm_n=1.0, seed=11),
              "indices": c1["indices"].tolist(),
              "weights": [[[round(float(x), 9) for x in r] for r in n] for n in c1["weights"]]}
    for name in ("out", "dq", "dk", "dv"):
        t = c1[name]
        digest[name] = {"sum": float(t.sum()), "abs_sum": float(t.abs().sum()), "max_abs": float(t.abs().max()),
                        "head": [float(x) for x in t.flatten()[:8]], "stride_sample": [float(x) for x in t.flatten()[::100003][:16]]}
    with open(os.path.join(HERE, "gca_cfg1_digest.json"), "w") as f:
        json.dump(digest, f, indent=1)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
