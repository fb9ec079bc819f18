// Reference lists of the indexed backward.
//
// Cache chunk cc = n*C + c is "referenced" by ref = z*K + j whenever indices[z, j] == c and row z
// belongs to sequence n.  The dk/dv kernels are chunk-centric: one workgroup sums the contributions
// of a chunk's references, so every cache gradient is written exactly once, in a fixed order, with
// no atomics on the gradients and no zero-fill.  The lists depend on the retrieval only (indices), not on a
// layer's tensors, so one build serves every layer that shares the retrieval.  Built on the device in one
// pass over the Z*K references (cost independent of the number of chunks per sequence):
//   zero     count[] = 0
//   count    one thread per reference: count[chunk]++
//   scan     one workgroup: exclusive scans giving each chunk its list start, its first segment, its first
//            partial slot and its first step in the stream (below); writes the segment table
//   scatter  one thread per reference: takes the next free place of its chunk's list
//   sort     one workgroup per chunk: sorts the list ascending, so the order the contributions are summed in is
//            fixed (and the run-to-run result bit-identical), and writes the (z, j) record of every entry
// A chunk's list is cut into segments of at most seg_max references, one dk/dv workgroup each (load balance:
// popular chunks can be referenced by every later query chunk).  A chunk with one segment (or none: then the
// segment is empty and the workgroup writes zeros) is stored directly; the segments of a longer list write float
// partial tiles to slots and a last small launch adds them up in segment order.
#pragma once
#include "gca_common.h"

namespace gca {

struct ListWs {
    int* count;       // [NC]       references per chunk
    int* start;       // [NC]       first position of the chunk's list in refs
    int* seg_base;    // [NC]       first segment of the chunk
    int* slot_base;   // [NC]       first partial slot of the chunk (only meaningful if it has > 1 segment)
    int* cursor;      // [NC]       scatter cursors
    int* nseg;        // [4]        [0] segments, [1] partial slots
    int* refs;        // [Z*K]      reference ids, chunk after chunk, ascending inside a chunk
    int* ref_zj;      // [2*Z*K]    (z, j) of refs[i] at [2i], [2i+1]: spares the kernels a division per reference
    int* seg_chunk;   // [bound]    chunk of the segment
    int* seg_start;   // [bound]    first position in refs
    int* seg_len;     // [bound]    references in the segment
    int* seg_slot;    // [bound]    partial slot, or -1 when the chunk has a single segment
    float* partials;  // [slots][Hkv][2][K_CTX*D] float
};

int64_t list_seg_bound(const Params& p, int seg_max);
int64_t list_slot_bound(const Params& p, int seg_max);
// bytes of the integer tables (what a build writes and a later call may reuse)
size_t list_table_bytes(const Params& p, int seg_max);
// tables + partial tiles
size_t list_ws_bytes(const Params& p, int seg_max);
// `tables` holds the integer tables, `partials` the float tiles (may be the bytes right after the tables)
ListWs list_carve(const Params& p, int seg_max, void* tables, void* partials);
// zero -> count -> scan -> scatter -> sort on stream s
int list_build(const Params& p, int seg_max, const int64_t* indices, const ListWs& ws, hipStream_t s);

__device__ __forceinline__ int64_t clamp_idx(int64_t c, int64_t C) { return c < 0 ? 0 : (c >= C ? C - 1 : c); }

}  // namespace gca
