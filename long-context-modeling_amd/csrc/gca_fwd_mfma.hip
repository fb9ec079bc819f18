// placeholder until the MFMA forward lands
#include "gca_common.h"
namespace gca {
bool mfma_supported(const gca_desc&) { return false; }
int launch_fwd_mfma(const gca_desc&, bool, const void*, const void*, const void*, const int64_t*, const void*, void*,
                    float*, hipStream_t) { return GCA_ERR_UNSUPPORTED; }
}
