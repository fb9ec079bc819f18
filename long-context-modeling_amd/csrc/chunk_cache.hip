// Append kernel of the device-resident chunk cache: new chunks are copied into their slots of a cache
// allocated with spare capacity, with the landmark row of every chunk kept, zeroed or dropped on the way.
// Pure data movement, bound by HBM: every workgroup moves 16-byte vectors, consecutive lanes touching
// consecutive addresses on both sides.
#include "gca_common.h"
#include "gca_mfma.h"

namespace gca {

namespace {

struct AppendArgs {
    int64_t N, capacity, count, n_new;
    int64_t src_chunk;    // elements per source chunk       (S or S+1) * Dm
    int64_t dst_chunk;    // elements per stored chunk       S * Dm
    int64_t copy_elems;   // leading elements of a chunk that are copied verbatim
    int64_t Dl;
};

// V = elements per 16-byte vector when everything is 16-byte aligned, else 1 (element-wise).
template <typename E, int V>
__global__ void __launch_bounds__(256)
chunk_append_kernel(AppendArgs a, const E* __restrict__ src_k, const E* __restrict__ src_v, const E* __restrict__ src_l,
                    E* __restrict__ dst_k, E* __restrict__ dst_v, E* __restrict__ dst_l) {
    // blockIdx.x = n * n_new + i (one appended chunk); the blockIdx.y workgroups of a chunk stride over its vectors
    const int64_t ci = blockIdx.x;
    const int64_t n = ci / a.n_new, i = ci % a.n_new;
    const int64_t slot = n * a.capacity + a.count + i;
    const E* sk = src_k + ci * a.src_chunk;
    const E* sv = src_v + ci * a.src_chunk;
    E* dk = dst_k + slot * a.dst_chunk;
    E* dv = dst_v + slot * a.dst_chunk;
    const int64_t nvec = a.dst_chunk / V, ncopy = a.copy_elems / V;
    for (int64_t t = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; t < nvec; t += (int64_t)gridDim.y * blockDim.x) {
        if (V == 1) {
            const E zero{};
            dk[t] = t < ncopy ? sk[t] : zero;
            dv[t] = t < ncopy ? sv[t] : zero;
        } else {
            u32x4 vk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
            if (t < ncopy) {
                vk = reinterpret_cast<const u32x4*>(sk)[t];
                vv = reinterpret_cast<const u32x4*>(sv)[t];
            }
            reinterpret_cast<u32x4*>(dk)[t] = vk;
            reinterpret_cast<u32x4*>(dv)[t] = vv;
        }
    }
    if (src_l != nullptr && blockIdx.y == 0) {
        for (int64_t t = threadIdx.x; t < a.Dl; t += blockDim.x) dst_l[slot * a.Dl + t] = src_l[ci * a.Dl + t];
    }
}

template <typename E>
int launch_append_t(const chunk_cache_desc& d, const AppendArgs& a, const void* sk, const void* sv, const void* sl,
                    void* dk, void* dv, void* dl, hipStream_t s) {
    constexpr int V = 16 / sizeof(E);
    const uintptr_t ptrs = (uintptr_t)sk | (uintptr_t)sv | (uintptr_t)dk | (uintptr_t)dv;
    const bool vec = ptrs % 16 == 0 && a.src_chunk % V == 0 && a.dst_chunk % V == 0 && a.copy_elems % V == 0;
    const int64_t nvec = vec ? a.dst_chunk / V : a.dst_chunk;
    int64_t by = (nvec + 255) / 256;   // workgroups per chunk
    if (by > 64) by = 64;
    if (by < 1) by = 1;
    const int64_t chunks = a.N * a.n_new;
    if (chunks > INT32_MAX) return GCA_ERR_SHAPE;
    const dim3 grid((unsigned)chunks, (unsigned)by);
    if (vec)
        hipLaunchKernelGGL((chunk_append_kernel<E, V>), grid, dim3(256), 0, s, a, (const E*)sk, (const E*)sv, (const E*)sl,
                           (E*)dk, (E*)dv, (E*)dl);
    else
        hipLaunchKernelGGL((chunk_append_kernel<E, 1>), grid, dim3(256), 0, s, a, (const E*)sk, (const E*)sv, (const E*)sl,
                           (E*)dk, (E*)dv, (E*)dl);
    return hipGetLastError() == hipSuccess ? GCA_OK : GCA_ERR_LAUNCH;
}

}  // namespace

int launch_chunk_append(const chunk_cache_desc& d, const void* sk, const void* sv, const void* sl,
                        void* dk, void* dv, void* dl, hipStream_t s) {
    AppendArgs a;
    a.N = d.N; a.capacity = d.capacity; a.count = d.count; a.n_new = d.n_new;
    a.dst_chunk = (int64_t)d.S * d.Dm;
    a.src_chunk = (int64_t)(d.lmk_row == CHUNK_LMK_DROP ? d.S + 1 : d.S) * d.Dm;
    a.copy_elems = (int64_t)(d.lmk_row == CHUNK_LMK_ZERO ? d.S - 1 : d.S) * d.Dm;
    a.Dl = d.Dl;
    if (d.dtype == GCA_F32) return launch_append_t<float>(d, a, sk, sv, sl, dk, dv, dl, s);
    if (d.dtype == GCA_BF16) return launch_append_t<uint16_t>(d, a, sk, sv, sl, dk, dv, dl, s);
    return GCA_ERR_DTYPE;
}

}  // namespace gca
