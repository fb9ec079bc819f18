#include <climits>
#include "gca_lists.h"

namespace gca {

int64_t list_seg_bound(const Params& p, int seg_max) { return p.N * p.C + (p.Z * p.K + seg_max - 1) / seg_max; }
int64_t list_slot_bound(const Params& p, int seg_max) { return 2 * ((p.Z * p.K + seg_max - 1) / seg_max) + 1; }

static size_t align256(size_t x) { return (x + 255) / 256 * 256; }

size_t list_table_bytes(const Params& p, int seg_max) {
    const size_t ints = (size_t)(5 * p.N * p.C + 4 + 3 * p.Z * p.K + 4 * list_seg_bound(p, seg_max));
    return align256(ints * sizeof(int));
}

size_t list_ws_bytes(const Params& p, int seg_max) {
    const size_t tile = (size_t)p.K_CTX * p.D;
    return list_table_bytes(p, seg_max) + (size_t)list_slot_bound(p, seg_max) * p.Hkv * 2 * tile * sizeof(float);
}

ListWs list_carve(const Params& p, int seg_max, void* tables, void* partials) {
    ListWs ws;
    int* base = (int*)tables;
    const int64_t NC = p.N * p.C, sb = list_seg_bound(p, seg_max);
    ws.count = base; base += NC;
    ws.start = base; base += NC;
    ws.seg_base = base; base += NC;
    ws.slot_base = base; base += NC;
    ws.cursor = base; base += NC;
    ws.nseg = base; base += 4;
    ws.refs = base; base += p.Z * p.K;
    ws.ref_zj = base; base += 2 * p.Z * p.K;
    ws.seg_chunk = base; base += sb;
    ws.seg_start = base; base += sb;
    ws.seg_len = base; base += sb;
    ws.seg_slot = base;
    ws.partials = (float*)partials;
    return ws;
}

__global__ void __launch_bounds__(256) gca_list_zero_kernel(int64_t n, int* __restrict__ a) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) a[i] = 0;
}

// chunk (global id n*C + c) that reference r = z*K + j points at
__device__ __forceinline__ int ref_chunk(const Params& p, const int64_t* __restrict__ indices, int64_t r) {
    const int64_t n = (r / p.K) / p.zpn;
    return (int)(n * p.C + clamp_idx(indices[r], p.C));
}

// one thread per reference.  SCATTER = false: count.  SCATTER = true: place the reference in its chunk's list
// (any order; the sort kernel fixes it).
template <bool SCATTER>
__global__ void __launch_bounds__(256)
gca_list_ref_kernel(Params p, const int64_t* __restrict__ indices, ListWs ws) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= p.Z * p.K) return;
    const int cc = ref_chunk(p, indices, r);
    if (!SCATTER) {
        atomicAdd(ws.count + cc, 1);
    } else {
        const int at = atomicAdd(ws.cursor + cc, 1);
        ws.refs[ws.start[cc] + at] = (int)r;
    }
}

// One workgroup: exclusive scans of the reference counts, the segment counts and the slot counts; writes each
// chunk's rows of the segment table and clears its scatter cursor.
__global__ void __launch_bounds__(1024)
gca_list_scan_kernel(Params p, int seg_max, ListWs ws) {
    __shared__ int s_a[1024], s_b[1024], s_c[1024];
    __shared__ int carry[4];
    const int tid = threadIdx.x;
    const int64_t NC = p.N * p.C;
    if (tid < 4) carry[tid] = 0;
    __syncthreads();
    for (int64_t base = 0; base < NC; base += 1024) {
        const int64_t cc = base + tid;
        const int cnt = cc < NC ? ws.count[cc] : 0;
        const int sg = cc < NC ? max(1, (cnt + seg_max - 1) / seg_max) : 0;
        const int sl = sg > 1 ? sg : 0;
        s_a[tid] = cnt; s_b[tid] = sg; s_c[tid] = sl;
        __syncthreads();
        for (int off = 1; off < 1024; off <<= 1) {
            const int a = tid >= off ? s_a[tid - off] : 0;
            const int b = tid >= off ? s_b[tid - off] : 0;
            const int c3 = tid >= off ? s_c[tid - off] : 0;
            __syncthreads();
            s_a[tid] += a; s_b[tid] += b; s_c[tid] += c3;
            __syncthreads();
        }
        if (cc < NC) {
            const int start = carry[0] + s_a[tid] - cnt;
            const int sb = carry[1] + s_b[tid] - sg;
            const int slot0 = carry[2] + s_c[tid] - sl;
            ws.start[cc] = start;
            ws.seg_base[cc] = sb;
            ws.slot_base[cc] = slot0;
            ws.cursor[cc] = 0;
            for (int s = 0; s < sg; ++s) {
                const int len = max(0, min(seg_max, cnt - s * seg_max));
                ws.seg_chunk[sb + s] = (int)cc;
                ws.seg_start[sb + s] = start + s * seg_max;
                ws.seg_len[sb + s] = len;
                ws.seg_slot[sb + s] = sg > 1 ? slot0 + s : -1;
            }
        }
        __syncthreads();
        if (tid == 1023) { carry[0] += s_a[1023]; carry[1] += s_b[1023]; carry[2] += s_c[1023]; }
        __syncthreads();
    }
    if (tid == 0) { ws.nseg[0] = carry[1]; ws.nseg[1] = carry[2]; }
}

// Ascending sort of a[0, n) by all threads of the workgroup: bitonic network in the form whose compare-exchanges
// all point the same way, so the padding up to the next power of two never has to be stored.
__device__ void sort_ascending(int* a, int n, int tid, int nt) {
    int P = 1;
    while (P < n) P <<= 1;
    for (int k = 2; k <= P; k <<= 1) {
        for (int j = k >> 1; j > 0; j >>= 1) {
            __syncthreads();
            for (int i = tid; i < P; i += nt) {
                const int l = (j == (k >> 1)) ? (i ^ (k - 1)) : (i ^ j);
                if (l > i && l < n) {
                    const int x = a[i], y = a[l];
                    if (x > y) { a[i] = y; a[l] = x; }
                }
            }
        }
    }
    __syncthreads();
}

// One workgroup per chunk: lists of up to SORT_LDS references are sorted in LDS, longer ones in place; then the
// (z, j) records of the list are written.
constexpr int SORT_LDS = 4096;
__global__ void __launch_bounds__(256)
gca_list_sort_kernel(Params p, ListWs ws) {
    __shared__ int buf[SORT_LDS];
    const int64_t cc = blockIdx.x;
    const int n = ws.count[cc];
    if (n == 0) return;
    const int start = ws.start[cc];
    int* list = ws.refs + start;
    const int tid = threadIdx.x;
    if (n >= 2 && n <= SORT_LDS) {
        for (int i = tid; i < n; i += 256) buf[i] = list[i];
        sort_ascending(buf, n, tid, 256);
        for (int i = tid; i < n; i += 256) list[i] = buf[i];
    } else if (n >= 2) {
        sort_ascending(list, n, tid, 256);
    }
    __syncthreads();
    for (int i = tid; i < n; i += 256) {
        const int ref = list[i];
        const int z = ref / p.K;
        ws.ref_zj[2 * (int64_t)(start + i)] = z;
        ws.ref_zj[2 * (int64_t)(start + i) + 1] = ref - z * p.K;
    }
}

int list_build(const Params& p, int seg_max, const int64_t* indices, const ListWs& ws, hipStream_t s) {
    const int64_t NC = p.N * p.C, R = p.Z * p.K;
    // every table entry is a 32-bit int: reference ids, chunk ids, list positions, segment numbers
    if (NC > INT_MAX || R > INT_MAX || list_seg_bound(p, seg_max) > INT_MAX) return GCA_ERR_SHAPE;
    const unsigned rb = (unsigned)((R + 255) / 256);
    hipLaunchKernelGGL(gca_list_zero_kernel, dim3((unsigned)((NC + 255) / 256)), dim3(256), 0, s, NC, ws.count);
    hipLaunchKernelGGL((gca_list_ref_kernel<false>), dim3(rb), dim3(256), 0, s, p, indices, ws);
    hipLaunchKernelGGL(gca_list_scan_kernel, dim3(1), dim3(1024), 0, s, p, seg_max, ws);
    hipLaunchKernelGGL((gca_list_ref_kernel<true>), dim3(rb), dim3(256), 0, s, p, indices, ws);
    hipLaunchKernelGGL(gca_list_sort_kernel, dim3((unsigned)NC), dim3(256), 0, s, p, ws);
    return hipGetLastError() == hipSuccess ? GCA_OK : GCA_ERR_LAUNCH;
}

}  // namespace gca
