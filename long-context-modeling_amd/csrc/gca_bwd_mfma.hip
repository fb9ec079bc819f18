// placeholder until the MFMA backward lands
#include "gca_common.h"
namespace gca {
int launch_bwd_mfma(const gca_desc&, bool, const void*, const void*, const void*, const int64_t*, const void*,
                    const void*, const float*, void*, void*, void*, float*, float*, hipStream_t) { return GCA_ERR_UNSUPPORTED; }
}
