#!/usr/bin/env python3
"""GCA hot-path benchmark on one MI355X.

A "step" is one GCA layer pass over one synthetic batch, everything resident in HBM:
landmark scoring + top-k + retrieval weights, indexed forward, indexed backward
(dq, cache-shaped dk/dv, dw).  The workload is BASELINE.json's config 2:
B=8, H=12, d=64, L=16384 (256 chunks of 64), top-k 8, bf16, softmax-off-by-one on.

Prints ONE JSON line: tokens/s of the whole step, plus
  roofline      the slowest kernel of the step timed on its own with HIP events on the launch
                stream, against the 8 TB/s HBM peak, with the algorithmic bytes of that kernel
  cpu_baseline  the CPU oracle (PyTorch einsum formulation + autograd) on BASELINE.json's
                config 1, timed on this host's cores
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "long-context-modeling_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_inputs(torch, dev, seed, N, C, H, S, d):
    """Config-2 synthetic data: q, K, V ~ N(0,1)*0.5; landmark keys = per-chunk mean of K + N(0, 0.1);
    landmark queries ~ N(0,1); grad_output ~ N(0,1)."""
    g = torch.Generator(device=dev).manual_seed(seed)
    Z = N * (C - 1)
    q = (torch.randn(Z, H, S, d, device=dev, generator=g) * 0.5).bfloat16().requires_grad_(True)
    ck = (torch.randn(N, C, S, H * d, device=dev, generator=g) * 0.5).bfloat16().requires_grad_(True)
    cv = (torch.randn(N, C, S, H * d, device=dev, generator=g) * 0.5).bfloat16().requires_grad_(True)
    lk = (ck.detach().float().mean(2) + 0.1 * torch.randn(N, C, H * d, device=dev, generator=g)).bfloat16()
    lq = torch.randn(N, C, H * d, device=dev, generator=g).bfloat16()
    do = torch.randn(Z, H, S, d, device=dev, generator=g).bfloat16()
    return q, ck, cv, lq, lk, do


def event_time(torch, fn, iters, warmup=2):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters   # ms


def kernel_times(torch, q, ck, cv, idx, w, do, sm_scale, sm_n, iters):
    """Times the forward launch and each backward stage on their own through the C ABI."""
    from gca_hip import _lib
    from gca_hip.gca import _desc, _ptr, _stream
    L = _lib.lib()
    dev = q.device
    N, C, S, Dm = ck.shape
    Z, H, _, d = q.shape
    K = idx.shape[1]
    o = torch.empty_like(q)
    lse = torch.empty((Z, H, K, S), device=dev, dtype=torch.float32)
    dq = torch.empty_like(q)
    dkc, dvc = torch.empty_like(ck), torch.empty_like(cv)
    dw = torch.empty((Z, K), device=dev, dtype=torch.float32)
    stream = _stream(dev)

    def desc(stages=0):
        dsc = _desc(q, K, S, Dm // d, w, sm_scale, sm_n, N=N, C=C)
        dsc.stages = stages
        return dsc

    nbytes = L.gca_bwd_workspace_bytes(ctypes.byref(desc()))
    ws = torch.empty(nbytes // 4 + 1, device=dev, dtype=torch.float32)

    def fwd():
        _lib.check(L.gca_fwd_indexed(ctypes.byref(desc()), _ptr(q), _ptr(ck), _ptr(cv), _ptr(idx), _ptr(w), _ptr(o),
                                     _ptr(lse), stream), "gca_fwd_indexed")

    def bwd(stages):
        def run():
            _lib.check(L.gca_bwd_indexed(ctypes.byref(desc(stages)), _ptr(q), _ptr(ck), _ptr(cv), _ptr(idx), _ptr(w),
                                         _ptr(do), _ptr(lse), _ptr(dq), _ptr(dkc), _ptr(dvc), _ptr(dw), _ptr(ws), nbytes,
                                         stream), "gca_bwd_indexed")
        return run

    fwd()
    bwd(0)()
    times = {
        "gca_fwd_mfma_kernel": event_time(torch, fwd, iters),
        "gca_bwd_dq_mfma_kernel": event_time(torch, bwd(1), iters),
        "gca_bwd_dkdv_mfma_kernel(+lists)": event_time(torch, bwd(2), iters),
        "gca_bwd_dw_kernel": event_time(torch, bwd(4), iters),
    }
    return times


def cpu_baseline(torch, budget_s=12.0):
    """CPU oracle at BASELINE.json config 1 (fp32, B=2, H=4, d=64, L=1024, chunk 64, top-k 4, softmax1 on):
    retrieval + forward + autograd backward, median over the iterations that fit the budget."""
    from oracle import gca_oracle as orc
    cores = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    N, C, H, S, d, K = 2, 16, 4, 64, 64, 4
    q_all = (torch.randn(N, C, H, S, d) * 0.5).requires_grad_(True)
    ck = (torch.randn(N, C, S, H * d) * 0.5).requires_grad_(True)
    cv = (torch.randn(N, C, S, H * d) * 0.5).requires_grad_(True)
    lq, lk = torch.randn(N, C, H * d), torch.randn(N, C, H * d)
    do = torch.randn(N, C, H, S, d)

    def step():
        out, _, _ = orc.gca_layer(q_all, ck, cv, lq, lk, K, H, sm_n=1.0)
        torch.autograd.grad(out, (q_all, ck, cv), do)

    for _ in range(3):
        step()
    ts = []
    t_end = time.perf_counter() + budget_s
    while (time.perf_counter() < t_end and len(ts) < 2000) or len(ts) < 10:
        t0 = time.perf_counter()
        step()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    med = ts[len(ts) // 2]
    return {"value": N * C * S / med, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"config 1 (fp32 B=2 H=4 d=64 L=1024 chunk=64 top-k=4), median of {len(ts)} fwd+bwd steps, "
                      f"{med * 1e3:.2f} ms/step, torch {torch.__version__}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--sm-n", type=float, default=1.0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (sharding is described in DESIGN.md)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import gca_hip

    dev = torch.device("cuda:0")
    N, C, H, S, d, K = 8, 256, 12, 64, 64, 8
    L_tokens = C * S
    sm_scale = 1.0 / math.sqrt(d)
    log(f"workload cfg2: B={N} H={H} d={d} L={L_tokens} chunk={S} top-k={K} bf16 sm_n={args.sm_n} seed={args.seed}")
    q, ck, cv, lq, lk, do = make_inputs(torch, dev, args.seed, N, C, H, S, d)
    Z = N * (C - 1)

    def step():
        _, indices, weights = gca_hip.landmark_retrieve(lq, lk, K, H * d)
        idx = indices[:, :-1].reshape(Z, -1).contiguous()
        w = weights[:, :-1].reshape(Z, -1).contiguous().requires_grad_(True)
        o = gca_hip.attention_indexed(q, ck, cv, idx, w, sm_scale, args.sm_n)
        return torch.autograd.grad(o, (q, ck, cv, w), do)

    if args.copy_calibration:
        src = torch.empty(1 << 29, device=dev, dtype=torch.bfloat16).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    tokens = N * L_tokens
    value = tokens / dt

    # per-kernel timing for the roofline entry (HIP events on the launch stream)
    _, indices, weights = gca_hip.landmark_retrieve(lq, lk, K, H * d)
    idx = indices[:, :-1].reshape(Z, -1).contiguous()
    w = weights[:, :-1].reshape(Z, -1).contiguous()
    kt = kernel_times(torch, q.detach(), ck.detach(), cv.detach(), idx, w, do, sm_scale, args.sm_n, max(args.steps, 10))
    t_retr = event_time(torch, lambda: gca_hip.landmark_retrieve(lq, lk, K, H * d), max(args.steps, 10))
    log("kernel times (ms): " + ", ".join(f"{k}={v:.3f}" for k, v in kt.items()) + f", retrieval={t_retr:.3f}")

    # algorithmic bytes per token (stream model: every query chunk streams its K retrieved chunks once)
    e = 2
    b_fwd = 2 * H * d * e + 2 * K * H * d * e + 4 * H * K
    b_dq = 2 * H * d * e + 4 * H * K + 2 * K * H * d * e + H * d * e          # q, dO, lse, gather, dq
    b_dkdv = 2 * K * H * d * 4                                                # fp32 dK/dV accumulation
    model = {"gca_fwd_mfma_kernel": b_fwd, "gca_bwd_dq_mfma_kernel": b_dq, "gca_bwd_dkdv_mfma_kernel(+lists)": b_dkdv}
    dom = max(model, key=lambda k_: kt[k_])
    achieved = model[dom] * tokens / (kt[dom] * 1e-3) / 1e9
    step_bytes = (b_fwd + b_dq + b_dkdv) * tokens
    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "kernel_ms": {k_: round(v, 4) for k_, v in kt.items()},
                "step_algorithmic_GB": round(step_bytes / 1e9, 3),
                "step_frac_of_hbm_roofline": round(step_bytes / dt / 1e9 / HBM_PEAK_GBS, 4)}

    out = {
        "metric": "GCA fwd+bwd tokens/s at L=16K (1 GPU)", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE config 2: GCA layer fwd+bwd incl. landmark retrieval, indexed kernels",
                   "batch": N, "heads": H, "head_dim": d, "seq_len": L_tokens, "chunk": S, "topk": K,
                   "softmax_off_by_one": args.sm_n},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
