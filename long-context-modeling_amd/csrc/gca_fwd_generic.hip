// Generic GCA forward: fp32 arithmetic on the vector ALUs for any supported shape and
// element type.  It is the fp32 path (1e-5 class accuracy), the decode path (Q_CTX of 1
// or 2) and the fallback for shapes the MFMA kernels do not take.
//
// Work split: one workgroup = 32 query rows of one (z, query head); 8 lanes share a row,
// each owning D/8 contiguous dims of q and of the output.  K/V tiles of KT key rows are
// staged in LDS as floats and shared by the 32 rows.  A score is a D/8-long partial dot
// product per lane followed by a 3-step butterfly over the 8 lanes, so every lane ends
// up with the whole score row and needs no further exchange for the softmax or P.V.
#include "gca_common.h"

namespace gca {

template <typename T, typename WT, int D>
__global__ void __launch_bounds__(256)
gca_fwd_generic_kernel(Params p, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                       const int64_t* __restrict__ indices, const WT* __restrict__ w,
                       T* __restrict__ o, float* __restrict__ lse) {
    constexpr int TPR = 8, QB = 32, DPT = D / TPR;
    constexpr int KT = (D >= 256) ? 16 : 32;
    __shared__ float sK[KT * D];
    __shared__ float sV[KT * D];

    const int tid = threadIdx.x;
    const int r = tid / TPR, t = tid % TPR;
    const int nqb = (p.Q_CTX + QB - 1) / QB;
    const int64_t bid = blockIdx.x;
    const int qb = (int)(bid % nqb);
    const int64_t zh = bid / nqb;
    const int h = (int)(zh % p.Hq);
    const int64_t z = zh / p.Hq;
    const int hk = h / p.G;
    const int row = qb * QB + r;
    const bool row_ok = row < p.Q_CTX;

    float qreg[DPT], acc[DPT];
#pragma unroll
    for (int i = 0; i < DPT; ++i) { qreg[i] = 0.f; acc[i] = 0.f; }
    if (row_ok) {
        const T* qp = q + q_base(p, z, h) + row * p.q_rs + t * DPT;
#pragma unroll
        for (int i = 0; i < DPT; ++i) qreg[i] = to_f(qp[i]);
    }
    const float c = p.sm_scale * LOG2E;

    for (int j = 0; j < p.K; ++j) {
        int64_t rs;
        const T* kj = chunk_base(p, k, indices, z, hk, j, rs);
        const T* vj = chunk_base(p, v, indices, z, hk, j, rs);
        // sm_n acts as sm_n extra keys with logit 0 and value 0.
        float m = (p.sm_n > 0.f) ? 0.f : -INFINITY;
        float l = (p.sm_n > 0.f) ? p.sm_n : 0.f;
        float oj[DPT];
#pragma unroll
        for (int i = 0; i < DPT; ++i) oj[i] = 0.f;

        for (int kt0 = 0; kt0 < p.K_CTX; kt0 += KT) {
            __syncthreads();
            for (int i = tid; i < KT * D; i += 256) {
                const int key = i / D, dd = i % D;
                const int gk = kt0 + key;
                float kv = 0.f, vv = 0.f;
                if (gk < p.K_CTX) {
                    kv = to_f(kj[(int64_t)gk * rs + dd]);
                    vv = to_f(vj[(int64_t)gk * rs + dd]);
                }
                sK[i] = kv;
                sV[i] = vv;
            }
            __syncthreads();
            const int nk = min(KT, p.K_CTX - kt0);
            float s[KT];
            float tmax = -INFINITY;
#pragma unroll
            for (int kk = 0; kk < KT; ++kk) {
                float part = 0.f;
#pragma unroll
                for (int i = 0; i < DPT; ++i) part = fmaf(qreg[i], sK[kk * D + t * DPT + i], part);
                part += __shfl_xor(part, 1);
                part += __shfl_xor(part, 2);
                part += __shfl_xor(part, 4);
                s[kk] = (kk < nk) ? part * c : -INFINITY;
                tmax = fmaxf(tmax, s[kk]);
            }
            const float m_new = fmaxf(m, tmax);
            const float alpha = (m == -INFINITY) ? 0.f : exp2f(m - m_new);
            l *= alpha;
#pragma unroll
            for (int i = 0; i < DPT; ++i) oj[i] *= alpha;
#pragma unroll
            for (int kk = 0; kk < KT; ++kk) {
                const float pe = exp2f(s[kk] - m_new);   // exp2(-inf) = 0 for the padded keys
                l += pe;
#pragma unroll
                for (int i = 0; i < DPT; ++i) oj[i] = fmaf(pe, sV[kk * D + t * DPT + i], oj[i]);
            }
            m = m_new;
        }
        const float wj = to_f(w[z * p.K + j]);
        const float inv = wj / l;
#pragma unroll
        for (int i = 0; i < DPT; ++i) acc[i] = fmaf(oj[i], inv, acc[i]);
        if (lse != nullptr && row_ok && t == 0)
            lse[((z * p.Hq + h) * (int64_t)p.K + j) * p.Q_CTX + row] = m + log2f(l);
    }
    if (row_ok) {
        T* op = o + q_base(p, z, h) + row * p.q_rs + t * DPT;
#pragma unroll
        for (int i = 0; i < DPT; ++i) op[i] = from_f<T>(acc[i]);
    }
}

template <typename T, typename WT, int D>
static int launch_d(const Params& p, const void* q, const void* k, const void* v, const int64_t* idx,
                    const void* w, void* o, float* lse, hipStream_t s) {
    const int nqb = (p.Q_CTX + 31) / 32;
    const int64_t blocks = p.Z * p.Hq * nqb;
    if (blocks <= 0 || blocks > 0x7fffffffLL) return GCA_ERR_SHAPE;
    hipLaunchKernelGGL((gca_fwd_generic_kernel<T, WT, D>), dim3((unsigned)blocks), dim3(256), 0, s, p,
                       (const T*)q, (const T*)k, (const T*)v, idx, (const WT*)w, (T*)o, lse);
    return hipGetLastError() == hipSuccess ? GCA_OK : GCA_ERR_LAUNCH;
}

template <typename T, typename WT>
static int launch_t(const Params& p, const void* q, const void* k, const void* v, const int64_t* idx,
                    const void* w, void* o, float* lse, hipStream_t s) {
    switch (p.D) {
        case 16: return launch_d<T, WT, 16>(p, q, k, v, idx, w, o, lse, s);
        case 32: return launch_d<T, WT, 32>(p, q, k, v, idx, w, o, lse, s);
        case 64: return launch_d<T, WT, 64>(p, q, k, v, idx, w, o, lse, s);
        case 128: return launch_d<T, WT, 128>(p, q, k, v, idx, w, o, lse, s);
        case 256: return launch_d<T, WT, 256>(p, q, k, v, idx, w, o, lse, s);
    }
    return GCA_ERR_SHAPE;
}

int launch_fwd_generic(const gca_desc& d, bool indexed, const void* q, const void* k, const void* v,
                       const int64_t* indices, const void* w, void* o, float* lse, hipStream_t s) {
    const Params p = make_params(d, indexed);
    if (d.dtype == GCA_F32 && d.w_dtype == GCA_F32) return launch_t<float, float>(p, q, k, v, indices, w, o, lse, s);
    if (d.dtype == GCA_F32 && d.w_dtype == GCA_BF16) return launch_t<float, bf16_t>(p, q, k, v, indices, w, o, lse, s);
    if (d.dtype == GCA_BF16 && d.w_dtype == GCA_F32) return launch_t<bf16_t, float>(p, q, k, v, indices, w, o, lse, s);
    if (d.dtype == GCA_BF16 && d.w_dtype == GCA_BF16) return launch_t<bf16_t, bf16_t>(p, q, k, v, indices, w, o, lse, s);
    return GCA_ERR_DTYPE;
}

}  // namespace gca
