// placeholder until the MFMA backward lands: the generic backward consumes the same lse
#include "gca_common.h"
namespace gca {
int launch_bwd_mfma(const gca_desc& d, bool indexed, const void* q, const void* k, const void* v, const int64_t* indices,
                    const void* w, const void* dout, const float* lse, void* dq, void* dk, void* dv, float* dw,
                    float* delta, hipStream_t s) {
    return launch_bwd_generic(d, indexed, q, k, v, indices, w, dout, lse, dq, dk, dv, dw, delta, s);
}
}
