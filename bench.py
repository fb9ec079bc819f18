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
# HBM bytes per launch of the three main kernels at config 2, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# scaled by the same counters' readings for a 1 GiB device copy (summary kept under profiles/)
MEASURED_TRAFFIC_GB = {"gca_fwd_mfma_kernel": 1.138, "gca_bwd_dq_mfma_kernel": 1.551, "gca_bwd_dkdv2_mfma_kernel": 1.776}


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
        "gca_list_build(3 launches)": event_time(torch, bwd(8), iters),
        "gca_bwd_dkdv2_mfma_kernel": event_time(torch, bwd(2), iters),
        "gca_bwd_dkdv_reduce_kernel": event_time(torch, bwd(16), iters),
        "gca_bwd_dw_kernel": event_time(torch, bwd(4), iters),
    }
    return times


def other_configs(torch, dev, seed):
    """BASELINE configs 3, 4, 5 on the same GPU: absolute tokens/s and the fraction of the binding
    (HBM) roofline from the stream-model bytes.  Forward-only configs time scoring + top-k + forward."""
    import gca_hip
    g = torch.Generator(device=dev).manual_seed(seed + 1)

    def rn(*shape, scale=1.0):
        return (torch.randn(*shape, device=dev, generator=g) * scale).bfloat16()

    out = {}
    # ---- config 4: GQA, wider heads, fwd+bwd.  Retrieval score logits ~ N(0,1) are given directly.
    N, C, Hq, Hkv, S, d, K = 4, 512, 32, 8, 64, 128, 16
    Z = N * (C - 1)
    q = rn(Z, Hq, S, d, scale=0.35).requires_grad_(True)
    do = rn(Z, Hq, S, d)
    ck = rn(N, C, S, Hkv * d, scale=0.35).requires_grad_(True)
    cv = rn(N, C, S, Hkv * d, scale=0.35).requires_grad_(True)
    scores = torch.randn(N, C, C, device=dev, generator=g).bfloat16()

    def step4():
        indices, weights = gca_hip.landmark_topk(scores, K)
        idx = indices[:, :-1].reshape(Z, K).contiguous()
        w = weights[:, :-1].reshape(Z, K).contiguous().requires_grad_(True)
        o = gca_hip.attention_indexed(q, ck, cv, idx, w, 1.0 / math.sqrt(d), 0.0)
        return torch.autograd.grad(o, (q, ck, cv, w), do)

    t = event_time(torch, step4, 5) * 1e-3
    tokens = N * C * S
    e = 2
    nbytes = (2 * Hq * d * e + 2 * K * Hkv * d * e + 4 * Hq * K) + (3 * Hq * d * e + 4 * Hq * K + 2 * K * Hkv * d * e + 2 * K * Hkv * d * 4)
    flops = 14 * Hq * K * S * d
    t_roof = max(nbytes * tokens / (HBM_PEAK_GBS * 1e9), flops * tokens / 2.5e15)
    out["cfg4_gqa_d128_fwd_bwd"] = {"tokens_per_s": round(tokens / t, 1), "ms": round(t * 1e3, 3),
                                    "frac_of_binding_roofline": round(t_roof / t, 4), "bound": "hbm",
                                    "algorithmic_TFLOP_per_s": round(flops * tokens / t / 1e12, 1)}
    del q, do, ck, cv, scores

    # ---- config 3: 1M-token prefill, forward only, one needle chunk with a 4x landmark
    N, C, H, S, d, K = 1, 16384, 12, 64, 64, 8
    Z = C - 1
    q = rn(Z, H, S, d, scale=0.5)
    ck, cv = rn(N, C, S, H * d, scale=0.5), rn(N, C, S, H * d, scale=0.5)
    lk = (ck.float().mean(2) + 0.1 * torch.randn(N, C, H * d, device=dev, generator=g)).bfloat16()
    lq = rn(N, C, H * d)
    needle = 4321
    lk[0, needle] = lk[0, needle] * 4 + lq[0, -1] * 0      # 4x norm at a fixed position
    lq = (lq + 0.5 * lk[0, needle]).bfloat16()            # queries correlate with the needle

    def step3():
        _, indices, weights = gca_hip.landmark_retrieve(lq, lk, K, H * d)
        idx = indices[:, :-1].reshape(Z, K).contiguous()
        w = weights[:, :-1].reshape(Z, K).contiguous()
        return gca_hip.gca_kv_cache_indexed(q, ck, cv, idx, w, 0.125, 1.0), indices

    _, indices = step3()
    hit = (indices[0, needle + 1:] == needle).any(-1).float().mean().item()
    t = event_time(torch, lambda: step3(), 3, 1) * 1e-3
    tokens = N * C * S
    nbytes = (2 * H * d * e + 2 * K * H * d * e + 4 * H * K) * tokens + 2 * N * C * H * d * e
    out["cfg3_prefill_1M_fwd"] = {"tokens_per_s": round(tokens / t, 1), "ms": round(t * 1e3, 3),
                                  "frac_of_binding_roofline": round(nbytes / (HBM_PEAK_GBS * 1e9) / t, 4), "bound": "hbm",
                                  "needle_selected_by_later_rows": round(hit, 4)}
    del q, ck, cv, lk, lq

    # ---- config 5: one decode chunk (64 new tokens) per sequence against a long cache
    for name, N, E in (("cfg5a_decode_B1_16M", 1, 262144), ("cfg5b_decode_B64_64K", 64, 1024)):
        H, S, d, K = 12, 64, 64, 8
        ck, cv = rn(N, E, S, H * d, scale=0.5), rn(N, E, S, H * d, scale=0.5)
        lk, lq = rn(N, E, H * d), rn(N, 1, H * d)
        q = rn(N, H, S, d, scale=0.5)

        def step5():
            _, indices, weights = gca_hip.landmark_retrieve(lq, lk, K, H * d)
            return gca_hip.gca_kv_cache_indexed(q, ck, cv, indices.view(N, K), weights.view(N, K), 0.125, 1.0)

        t = event_time(torch, step5, 20, 3) * 1e-3
        nbytes = N * E * H * d * e + N * (2 * K * S * H * d * e + 2 * H * S * d * e)
        out[name] = {"new_tokens_per_s": round(N * S / t, 1), "us": round(t * 1e6, 2),
                     "frac_of_binding_roofline": round(nbytes / (HBM_PEAK_GBS * 1e9) / t, 4), "bound": "hbm",
                     "scan_GB_per_s": None}
        t_scan = event_time(torch, lambda: gca_hip.landmark_scores(lq, lk, H * d), 20, 3) * 1e-3
        out[name]["scan_GB_per_s"] = round(N * E * H * d * e / t_scan / 1e9, 1)
        del ck, cv, lk, lq, q
    return out


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
    ap.add_argument("--all-configs", action="store_true",
                    help="also time BASELINE configs 3, 4 and 5 (adds an other_configs object to the JSON line)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (a kernel of known traffic, for scaling "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path is built)")

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
    model = {"gca_fwd_mfma_kernel": b_fwd, "gca_bwd_dq_mfma_kernel": b_dq, "gca_bwd_dkdv2_mfma_kernel": b_dkdv}
    dom = max(model, key=lambda k_: kt[k_])
    achieved = model[dom] * tokens / (kt[dom] * 1e-3) / 1e9
    step_bytes = (b_fwd + b_dq + b_dkdv) * tokens
    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": round(MEASURED_TRAFFIC_GB[dom] / (kt[dom] * 1e-3), 1),
                "traffic_GB_per_launch": MEASURED_TRAFFIC_GB[dom],
                "algorithmic_GB_per_launch": round(model[dom] * tokens / 1e9, 3),
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
    if args.all_configs:
        del q, ck, cv, lq, lk, do
        torch.cuda.empty_cache()
        out["other_configs"] = other_configs(torch, dev, args.seed)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
