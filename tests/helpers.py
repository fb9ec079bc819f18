"""Seeded input builders and error measures shared by the GPU parity tests."""
import math

import torch

from oracle import gca_oracle as orc


def gen(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def gca_inputs(Z, Hq, Hkv, K, Q, S, d, dtype, seed=0, scale=0.5, w_dtype=None):
    q = gen((Z, Hq, Q, d), seed, scale, dtype)
    k = gen((Z, Hkv, K, S, d), seed + 1, scale, dtype)
    v = gen((Z, Hkv, K, S, d), seed + 2, scale, dtype)
    g = torch.Generator().manual_seed(seed + 3)
    w = torch.softmax(torch.rand(Z, K, generator=g), -1).to(w_dtype or dtype)
    do = gen((Z, Hq, Q, d), seed + 4, 1.0, dtype)
    return q, k, v, w, do


def rel_err(got, ref):
    """max |got - ref| / max |ref|  (the "relative error" the tolerances below refer to)."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def oracle64(q, k, v, w, do, sm_scale, sm_n):
    """Oracle forward + explicit backward in float64 on exactly the given (already rounded) inputs."""
    q, k, v, w, do = [t.detach().double().cpu() for t in (q, k, v, w, do)]
    o = orc.gca_forward(q, k, v, w, sm_scale, sm_n)
    dq, dk, dv, dw = orc.gca_backward(q, k, v, w, do, sm_scale, sm_n)
    return o, dq, dk, dv, dw
