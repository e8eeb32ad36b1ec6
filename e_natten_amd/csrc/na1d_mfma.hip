// 1D matrix-core kernels for bf16 / fp16 sequences whose head dim is 32, 64 or 128 (the kernels
// of na1d_mfma_kernels.h built for exactly those dims); other multiples of 8 up to 128 are handed
// to the build in na1d_mfma_narrow.hip.
#include "na2d_common.h"

namespace enatten {
namespace {
constexpr bool kNarrow = false;
}
}  // namespace enatten

#include "na1d_mfma_kernels.h"

namespace enatten {

// bf16 / f16 sequences, head dims that are multiples of 8 up to 128, odd kernel_size 3 .. 49
bool mfma1d_supported(int D, int ks, int dtype) {
    return (dtype == ENATTEN_BF16 || dtype == ENATTEN_F16) && D >= 8 && D <= 128 && D % 8 == 0 &&
           ks >= 3 && ks <= 49 && ks % 2 == 1;
}

int launch_fwd1d_mfma(const FwdArgs &a, int dtype, hipStream_t st) {
    if (a.s.D != built_dim1(a.s.D)) return launch_fwd1d_mfma_narrow(a, dtype, st);
    return fwd1d_dispatch(a, dtype, st);
}

int launch_bwd1d_mfma(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    if (a.s.D != built_dim1(a.s.D)) return launch_bwd1d_mfma_narrow(a, dtype, path, st);
    return bwd1d_dispatch(a, dtype, path, st);
}

}  // namespace enatten
