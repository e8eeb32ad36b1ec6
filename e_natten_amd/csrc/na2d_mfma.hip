// Matrix-core (MFMA) kernels: placeholder until they are written.
#include "na2d_common.h"

namespace enatten {
bool mfma_supported(int, int, int) { return false; }
int launch_fwd_mfma(const FwdArgs &, int, hipStream_t) {
    set_error("matrix-core kernels are not built");
    return ENATTEN_EUNSUPPORTED;
}
int launch_bwd_mfma(const BwdArgs &, int, hipStream_t) {
    set_error("matrix-core kernels are not built");
    return ENATTEN_EUNSUPPORTED;
}
}  // namespace enatten
