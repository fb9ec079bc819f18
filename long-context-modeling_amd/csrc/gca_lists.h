// Reference lists of the indexed backward.
//
// Cache chunk cc = n*C + c is "referenced" by ref = z*K + j whenever indices[z, j] == c and row z
// belongs to sequence n.  The dk/dv kernels are chunk-centric: one workgroup sums the contributions
// of a chunk's references, so every cache gradient is written exactly once, in a fixed order, with
// no atomics and no zero-fill.  Lists are built on the device in three launches:
//   count  one wavefront per chunk sweeps the sequence's indices 64 at a time (ballot + popcount)
//   scan   one workgroup: exclusive scans giving each chunk its list start, its first segment and
//          its first partial slot
//   fill   same walk; a matching lane's rank in the ballot is its place in the list, so the reference
//          ids come out ascending per chunk; lane 0 writes the chunk's rows of the segment table
// A chunk's list is cut into segments of at most seg_max references, one dk/dv workgroup each
// (load balance: popular chunks can be referenced by every later query chunk).  A chunk with one
// segment (or none: then the segment is empty and the workgroup writes zeros) is stored directly;
// the segments of a longer list write float partial tiles to slots and a last small launch adds
// them up in segment order.
#pragma once
#include "gca_common.h"

namespace gca {

struct ListWs {
    int* count;       // [NC]     references per chunk
    int* start;       // [NC]     first position of the chunk's list in refs
    int* seg_base;    // [NC]     first segment of the chunk
    int* slot_base;   // [NC]     first partial slot of the chunk (only meaningful if it has > 1 segment)
    int* nseg;        // [4]      [0] total number of segments
    int* refs;        // [Z*K]    reference ids, chunk after chunk
    int* seg_chunk;   // [bound]  chunk of the segment
    int* seg_start;   // [bound]  first position in refs
    int* seg_len;     // [bound]  references in the segment
    int* seg_slot;    // [bound]  partial slot, or -1 when the chunk has a single segment
    float* partials;  // [slots][Hkv][2][K_CTX*D] float
};

int64_t list_seg_bound(const Params& p, int seg_max);
int64_t list_slot_bound(const Params& p, int seg_max);
size_t list_ws_bytes(const Params& p, int seg_max);
ListWs list_carve(const Params& p, int seg_max, void* base);
// count -> scan -> fill on stream s
int list_build(const Params& p, int seg_max, const int64_t* indices, const ListWs& ws, hipStream_t s);

__device__ __forceinline__ int64_t clamp_idx(int64_t c, int64_t C) { return c < 0 ? 0 : (c >= C ? C - 1 : c); }

}  // namespace gca
