// Matrix-core kernels for bf16 / fp16 tensors whose head dim is 32, 64 or 128: the kernels of
// na2d_mfma_kernels.h built for exactly those dims.  Other multiples of 8 up to 128 are handed
// to the build in na2d_mfma_narrow.hip.
#include "na2d_common.h"

namespace enatten {
namespace {
constexpr bool kNarrow = false;
}
}  // namespace enatten

#include "na2d_mfma_kernels.h"

namespace enatten {

// bf16 / fp16, head dims that are multiples of 8 up to 128, odd kernel sizes 3..13 whose halo
// fits LDS (all of them at the built dims 32, 64, 128).
bool mfma_supported(int D, int ks, int dtype) {
    if (dtype != ENATTEN_BF16 && dtype != ENATTEN_F16) return false;
    if (D < 8 || D > 128 || D % 8 != 0) return false;
    if (ks < 3 || ks > 13 || ks % 2 == 0) return false;
    const int DB = built_dim(D);
    // (head dims below 64 with kernel_size 11 and 13: the dK/dV pass of those lays its partial
    // sums over the staged rows, zeroed channels included)
    if (D != DB && DB == 64 && ks >= 11) return false;
    return fits_rt(DB, ks);
}

int launch_fwd_mfma(const FwdArgs &a, int dtype, hipStream_t st) {
    if (a.s.D != built_dim(a.s.D)) return launch_fwd_mfma_narrow(a, dtype, st);
    return fwd_dispatch(a, dtype, st);
}

int launch_bwd_mfma(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    if (a.s.D != built_dim(a.s.D)) return launch_bwd_mfma_narrow(a, dtype, path, st);
    return bwd_dispatch(a, dtype, path, st);
}

}  // namespace enatten
