// The 1D kernels of na1d_mfma_kernels.h built for head dims BELOW the one they are laid out for
// (any multiple of 8 runs on the kernels of the next of 32, 64, 128: the missing channels are zero
// in LDS and in the operand registers and are left out of the stores).
#include "na2d_common.h"

namespace enatten {
namespace {
constexpr bool kNarrow = true;
}
}  // namespace enatten

#include "na1d_mfma_kernels.h"

namespace enatten {

int launch_fwd1d_mfma_narrow(const FwdArgs &a, int dtype, hipStream_t st) {
    return fwd1d_dispatch(a, dtype, st);
}

int launch_bwd1d_mfma_narrow(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    return bwd1d_dispatch(a, dtype, path, st);
}

}  // namespace enatten
