// The kernels of na2d_mfma_kernels.h built for head dims BELOW the one they are laid out for:
// a head dim that is a multiple of 8 runs on the kernels of the next of 32, 64 and 128, with
// the missing channels zero in LDS and in the operand registers and left out of the stores.
// B4 N4 128x128 k5 bf16, forward+backward: head_dim 48 107 us (general kernels: 570), head_dim
// 96 213 us, head_dim 16 (16 heads) 225 us.
#include "na2d_common.h"

namespace enatten {
namespace {
constexpr bool kNarrow = true;
}
}  // namespace enatten

#include "na2d_mfma_kernels.h"

namespace enatten {

int launch_fwd_mfma_narrow(const FwdArgs &a, int dtype, hipStream_t st) {
    return fwd_dispatch(a, dtype, st);
}

int launch_bwd_mfma_narrow(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    return bwd_dispatch(a, dtype, path, st);
}

}  // namespace enatten
