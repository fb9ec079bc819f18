#include "gca_lists.h"

namespace gca {

int64_t list_seg_bound(const Params& p, int seg_max) { return p.N * p.C + (p.Z * p.K + seg_max - 1) / seg_max; }
int64_t list_slot_bound(const Params& p, int seg_max) { return 2 * ((p.Z * p.K + seg_max - 1) / seg_max) + 1; }

static size_t align256(size_t x) { return (x + 255) / 256 * 256; }

static size_t int_part_bytes(const Params& p, int seg_max) {
    const size_t ints = (size_t)(4 * p.N * p.C + 4 + p.Z * p.K + 4 * list_seg_bound(p, seg_max));
    return align256(ints * sizeof(int));
}

size_t list_ws_bytes(const Params& p, int seg_max) {
    const size_t tile = (size_t)p.K_CTX * p.D;
    return int_part_bytes(p, seg_max) + (size_t)list_slot_bound(p, seg_max) * p.Hkv * 2 * tile * sizeof(float);
}

ListWs list_carve(const Params& p, int seg_max, void* base_v) {
    ListWs ws;
    int* base = (int*)base_v;
    const int64_t NC = p.N * p.C, sb = list_seg_bound(p, seg_max);
    ws.count = base; base += NC;
    ws.start = base; base += NC;
    ws.seg_base = base; base += NC;
    ws.slot_base = base; base += NC;
    ws.nseg = base; base += 4;
    ws.refs = base; base += p.Z * p.K;
    ws.seg_chunk = base; base += sb;
    ws.seg_start = base; base += sb;
    ws.seg_len = base; base += sb;
    ws.seg_slot = base;
    ws.partials = (float*)((char*)base_v + int_part_bytes(p, seg_max));
    return ws;
}

// One wavefront per cache chunk: the lanes sweep the sequence's indices 64 at a time; a ballot gives
// the number of matches and each matching lane's rank, so lists come out ascending without sorting.
// grid (ceil(C/4), N), 256 threads.  FILL = false: count.  FILL = true: refs and the segment table.
template <bool FILL>
__global__ void __launch_bounds__(256)
gca_list_walk_kernel(Params p, int seg_max, const int64_t* __restrict__ indices, ListWs ws) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t n = blockIdx.y;
    const int64_t c = (int64_t)blockIdx.x * 4 + wave;
    if (c >= p.C) return;
    const int64_t cc = n * p.C + c;
    const int64_t nref = p.zpn * p.K;           // references of this sequence
    const int64_t r0 = n * nref;
    int cnt = 0;
    const int start = FILL ? ws.start[cc] : 0;
    const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll 4
    for (int64_t base = 0; base < nref; base += 64) {
        const int64_t i = base + lane;
        const bool match = i < nref && clamp_idx(indices[r0 + i], p.C) == c;
        const unsigned long long mask = __ballot(match);
        if (FILL && match) ws.refs[start + cnt + __popcll(mask & below)] = (int)(r0 + i);
        cnt += __popcll(mask);
    }
    if (lane != 0) return;
    if (!FILL) {
        ws.count[cc] = cnt;
    } else {
        const int sg = max(1, (cnt + seg_max - 1) / seg_max);
        const int sb = ws.seg_base[cc], slot0 = ws.slot_base[cc];
        for (int s = 0; s < sg; ++s) {
            ws.seg_chunk[sb + s] = (int)cc;
            ws.seg_start[sb + s] = start + s * seg_max;
            ws.seg_len[sb + s] = max(0, min(seg_max, cnt - s * seg_max));
            ws.seg_slot[sb + s] = sg > 1 ? slot0 + s : -1;
        }
    }
}

// one workgroup: exclusive scans of the reference counts, the segment counts and the slot counts
__global__ void __launch_bounds__(1024)
gca_list_scan_kernel(Params p, int seg_max, ListWs ws) {
    __shared__ int s_a[1024], s_b[1024], s_c[1024];
    __shared__ int carry[3];
    const int tid = threadIdx.x;
    const int64_t NC = p.N * p.C;
    if (tid < 3) carry[tid] = 0;
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
            ws.start[cc] = carry[0] + s_a[tid] - cnt;
            ws.seg_base[cc] = carry[1] + s_b[tid] - sg;
            ws.slot_base[cc] = carry[2] + s_c[tid] - sl;
        }
        __syncthreads();
        if (tid == 1023) { carry[0] += s_a[1023]; carry[1] += s_b[1023]; carry[2] += s_c[1023]; }
        __syncthreads();
    }
    if (tid == 0) { ws.nseg[0] = carry[1]; ws.nseg[1] = carry[2]; }
}

int list_build(const Params& p, int seg_max, const int64_t* indices, const ListWs& ws, hipStream_t s) {
    if (p.N > 65535) return GCA_ERR_SHAPE;
    const dim3 grid((unsigned)((p.C + 3) / 4), (unsigned)p.N);
    hipLaunchKernelGGL((gca_list_walk_kernel<false>), grid, dim3(256), 0, s, p, seg_max, indices, ws);
    hipLaunchKernelGGL(gca_list_scan_kernel, dim3(1), dim3(1024), 0, s, p, seg_max, ws);
    hipLaunchKernelGGL((gca_list_walk_kernel<true>), grid, dim3(256), 0, s, p, seg_max, indices, ws);
    return hipGetLastError() == hipSuccess ? GCA_OK : GCA_ERR_LAUNCH;
}

}  // namespace gca
