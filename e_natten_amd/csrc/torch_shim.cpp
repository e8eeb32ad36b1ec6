// Native torch binding of libenatten.so: the operators enatten::na{1,2}d_{fwd,bwd}
// and the differentiable enatten::natten{1,2}d, registered from C++ so that neither
// the forward nor the backward runs any Python.  (The backward of a Python
// autograd.Function is called on the autograd engine's device thread; measured per
// forward+backward on small inputs, the host side costs about 180 us that way and
// about a third of it from here.)  Host code only: tensors and streams come from
// torch, all device work goes through the C ABI in enatten.h.
//
// Same contract as the reference Functions (e_natten/triton.py:425-483 for 1D,
// :487-548 for 2D): q, k, v of one shape, dtype and device in, one tensor out,
// gradients for q, k and v only.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/library.h>

#include <tuple>

#include "enatten.h"

namespace {

using at::Tensor;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

int dtype_code(const Tensor &t) {
    switch (t.scalar_type()) {
        case at::kFloat: return ENATTEN_F32;
        case at::kBFloat16: return ENATTEN_BF16;
        case at::kHalf: return ENATTEN_F16;
        case at::kDouble: return ENATTEN_F64;
        default: return -1;
    }
}

// The checks of the Python host side, with the same error classes: ValueError for
// bad shapes, dtypes and kernel sizes, RuntimeError for tensors that are not on
// the GPU.
void validate(const char *what, const Tensor &q, const Tensor &k, const Tensor &v, int64_t ks,
              int64_t ndim) {
    TORCH_CHECK_VALUE(q.dim() == ndim, what, ": expected ",
                      ndim == 5 ? "[B, heads, H, W, head_dim]" : "[B, heads, T, head_dim]",
                      " tensors, got ", q.dim(), "-D q");
    TORCH_CHECK_VALUE(k.sizes() == q.sizes() && v.sizes() == q.sizes(), what,
                      ": q, k and v must have the same shape, got ", q.sizes(), ", ", k.sizes(),
                      ", ", v.sizes());
    TORCH_CHECK_VALUE(k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type(),
                      what, ": q, k and v must share a dtype");
    TORCH_CHECK_VALUE(dtype_code(q) >= 0, what, ": dtype ", q.scalar_type(),
                      " is not supported (float32, bfloat16, float16, float64)");
    TORCH_CHECK_VALUE(k.device() == q.device() && v.device() == q.device(), what,
                      ": q, k and v must be on the same device");
    TORCH_CHECK_VALUE(ks >= 1 && ks % 2 == 1, what, ": kernel_size must be odd and >= 1, got ", ks);
    for (int64_t d = 2; d < ndim - 1; d++)
        TORCH_CHECK_VALUE(q.size(d) >= ks, what, ": input of extent ", q.sizes().slice(2, ndim - 3),
                          " is smaller than kernel_size ", ks);
    TORCH_CHECK_VALUE(q.numel() > 0, what, ": empty tensors are not supported");
    TORCH_CHECK_VALUE(q.size(-1) <= 1024, what, ": head_dim ", q.size(-1),
                      " exceeds the supported maximum of 1024");
    // meta tensors (shape inference under tracing) pass: every operator returns outputs of
    // the right shape for them without touching the library
    TORCH_CHECK(q.is_cuda() || q.is_meta(), what,
                ": tensors must be on the GPU; this build has no CPU path");
}

// The kernels take any strides on the leading axes but need unit stride on the
// channel axis.
Tensor kernel_layout(const Tensor &t) {
    return (t.stride(-1) != 1 && t.size(-1) != 1) ? t.contiguous() : t;
}

void check_rc(int rc) {
    if (rc == ENATTEN_OK) return;
    const char *msg = enatten_last_error();
    TORCH_CHECK_VALUE(rc != ENATTEN_EINVAL, msg);
    TORCH_CHECK(false, msg);
}

void check_bwd_extras(const char *what, const Tensor &q, const Tensor &o, const Tensor &d_o) {
    TORCH_CHECK_VALUE(d_o.sizes() == q.sizes() && o.sizes() == q.sizes(), what,
                      ": o and d_o must have the shape of q");
    TORCH_CHECK_VALUE(d_o.scalar_type() == q.scalar_type() && o.scalar_type() == q.scalar_type(),
                      what, ": o and d_o must have the dtype of q");
}

std::tuple<Tensor, Tensor> na2d_fwd(const Tensor &q_, const Tensor &k_, const Tensor &v_,
                                    int64_t ks, double scale) {
    validate("enatten::na2d_fwd", q_, k_, v_, ks, 5);
    if (q_.is_meta())
        return {at::empty_like(kernel_layout(q_)),
                at::empty({q_.size(0), q_.size(1), q_.size(2), q_.size(3)}, q_.options().dtype(at::kFloat))};
    const c10::DeviceGuard guard(q_.device());
    const Tensor q = kernel_layout(q_), k = kernel_layout(k_), v = kernel_layout(v_);
    const int B = q.size(0), N = q.size(1), H = q.size(2), W = q.size(3), D = q.size(4);
    // like the reference's zeros_like(Q) (e_natten/triton.py:502) the output takes the
    // memory order of q
    Tensor o = kernel_layout(at::empty_like(q));
    Tensor lse = at::empty({B, N, H, W}, q.options().dtype(at::kFloat));
    check_rc(enatten2d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                           lse.data_ptr<float>(), B, N, H, W, D, (int)ks, dtype_code(q),
                           q.strides().data(), k.strides().data(), v.strides().data(),
                           o.strides().data(), (float)scale,
                           c10::hip::getCurrentHIPStream().stream()));
    return {o, lse};
}

std::tuple<Tensor, Tensor, Tensor> na2d_bwd(const Tensor &q_, const Tensor &k_, const Tensor &v_,
                                            const Tensor &o_, const Tensor &lse_,
                                            const Tensor &d_o_, int64_t ks, double scale) {
    validate("enatten::na2d_bwd", q_, k_, v_, ks, 5);
    check_bwd_extras("enatten::na2d_bwd", q_, o_, d_o_);
    if (q_.is_meta()) {
        const Tensor g = at::empty(q_.sizes(), q_.options());
        return {g, at::empty_like(g), at::empty_like(g)};
    }
    const c10::DeviceGuard guard(q_.device());
    const Tensor q = kernel_layout(q_), k = kernel_layout(k_), v = kernel_layout(v_);
    const Tensor o = kernel_layout(o_), d_o = kernel_layout(d_o_), lse = lse_.contiguous();
    const int B = q.size(0), N = q.size(1), H = q.size(2), W = q.size(3), D = q.size(4);
    Tensor dq = at::empty({B, N, H, W, D}, q.options());
    Tensor dk = at::empty_like(dq), dv = at::empty_like(dq);
    Tensor ws = at::empty({(int64_t)enatten2d_bwd_workspace_bytes(B, N, H, W, D, (int)ks, dtype_code(q))},
                          q.options().dtype(at::kByte));
    check_rc(enatten2d_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                           lse.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                           ws.data_ptr(), B, N, H, W, D, (int)ks, dtype_code(q),
                           q.strides().data(), k.strides().data(), v.strides().data(),
                           o.strides().data(), d_o.strides().data(), (float)scale,
                           c10::hip::getCurrentHIPStream().stream()));
    return {dq, dk, dv};
}

std::tuple<Tensor, Tensor> na1d_fwd(const Tensor &q_, const Tensor &k_, const Tensor &v_,
                                    int64_t ks, double scale) {
    validate("enatten::na1d_fwd", q_, k_, v_, ks, 4);
    if (q_.is_meta())
        return {at::empty_like(kernel_layout(q_)),
                at::empty({q_.size(0), q_.size(1), q_.size(2)}, q_.options().dtype(at::kFloat))};
    const c10::DeviceGuard guard(q_.device());
    const Tensor q = kernel_layout(q_), k = kernel_layout(k_), v = kernel_layout(v_);
    const int B = q.size(0), N = q.size(1), T = q.size(2), D = q.size(3);
    Tensor o = kernel_layout(at::empty_like(q));
    Tensor lse = at::empty({B, N, T}, q.options().dtype(at::kFloat));
    check_rc(enatten1d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                           lse.data_ptr<float>(), B, N, T, D, (int)ks, dtype_code(q),
                           q.strides().data(), k.strides().data(), v.strides().data(),
                           o.strides().data(), (float)scale,
                           c10::hip::getCurrentHIPStream().stream()));
    return {o, lse};
}

std::tuple<Tensor, Tensor, Tensor> na1d_bwd(const Tensor &q_, const Tensor &k_, const Tensor &v_,
                                            const Tensor &o_, const Tensor &lse_,
                                            const Tensor &d_o_, int64_t ks, double scale) {
    validate("enatten::na1d_bwd", q_, k_, v_, ks, 4);
    check_bwd_extras("enatten::na1d_bwd", q_, o_, d_o_);
    if (q_.is_meta()) {
        const Tensor g = at::empty(q_.sizes(), q_.options());
        return {g, at::empty_like(g), at::empty_like(g)};
    }
    const c10::DeviceGuard guard(q_.device());
    const Tensor q = kernel_layout(q_), k = kernel_layout(k_), v = kernel_layout(v_);
    const Tensor o = kernel_layout(o_), d_o = kernel_layout(d_o_), lse = lse_.contiguous();
    const int B = q.size(0), N = q.size(1), T = q.size(2), D = q.size(3);
    Tensor dq = at::empty({B, N, T, D}, q.options());
    Tensor dk = at::empty_like(dq), dv = at::empty_like(dq);
    Tensor ws = at::empty({(int64_t)enatten1d_bwd_workspace_bytes(B, N, T)},
                          q.options().dtype(at::kByte));
    check_rc(enatten1d_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                           lse.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                           ws.data_ptr(), B, N, T, D, (int)ks, dtype_code(q), q.strides().data(),
                           k.strides().data(), v.strides().data(), o.strides().data(),
                           d_o.strides().data(), (float)scale,
                           c10::hip::getCurrentHIPStream().stream()));
    return {dq, dk, dv};
}

// The composite operators reach the four kernels' operators through the dispatcher, not
// by a C++ call: tensor subclasses and modes above the backend keys (fake tensors under
// torch.compile, functorch wrappers) then see them as opaque operators with a meta kernel.
std::tuple<Tensor, Tensor> call_fwd(bool two_d, const Tensor &q, const Tensor &k, const Tensor &v,
                                    int64_t ks, double scale) {
    using Sig = std::tuple<Tensor, Tensor>(const Tensor &, const Tensor &, const Tensor &, int64_t,
                                           double);
    static const auto op2 =
        c10::Dispatcher::singleton().findSchemaOrThrow("enatten::na2d_fwd", "").typed<Sig>();
    static const auto op1 =
        c10::Dispatcher::singleton().findSchemaOrThrow("enatten::na1d_fwd", "").typed<Sig>();
    return (two_d ? op2 : op1).call(q, k, v, ks, scale);
}
std::tuple<Tensor, Tensor, Tensor> call_bwd(bool two_d, const Tensor &q, const Tensor &k,
                                            const Tensor &v, const Tensor &o, const Tensor &lse,
                                            const Tensor &d_o, int64_t ks, double scale) {
    using Sig = std::tuple<Tensor, Tensor, Tensor>(const Tensor &, const Tensor &, const Tensor &,
                                                   const Tensor &, const Tensor &, const Tensor &,
                                                   int64_t, double);
    static const auto op2 =
        c10::Dispatcher::singleton().findSchemaOrThrow("enatten::na2d_bwd", "").typed<Sig>();
    static const auto op1 =
        c10::Dispatcher::singleton().findSchemaOrThrow("enatten::na1d_bwd", "").typed<Sig>();
    return (two_d ? op2 : op1).call(q, k, v, o, lse, d_o, ks, scale);
}

// One autograd node for both operators: the forward keeps (q, k, v, o, lse), the
// backward returns (dQ, dK, dV) and no gradient for kernel_size and scale.
template <bool TWO_D>
struct NattenFn : public torch::autograd::Function<NattenFn<TWO_D>> {
    static Tensor forward(AutogradContext *ctx, const Tensor &q, const Tensor &k, const Tensor &v,
                          int64_t ks, double scale) {
        at::AutoDispatchBelowADInplaceOrView below;
        Tensor o, lse;
        std::tie(o, lse) = call_fwd(TWO_D, q, k, v, ks, scale);
        ctx->save_for_backward({q, k, v, o, lse});
        ctx->saved_data["kernel_size"] = ks;
        ctx->saved_data["scale"] = scale;
        return o;
    }
    static variable_list backward(AutogradContext *ctx, variable_list grads) {
        const variable_list s = ctx->get_saved_variables();
        const int64_t ks = ctx->saved_data["kernel_size"].toInt();
        const double scale = ctx->saved_data["scale"].toDouble();
        at::AutoDispatchBelowADInplaceOrView below;
        Tensor dq, dk, dv;
        std::tie(dq, dk, dv) = call_bwd(TWO_D, s[0], s[1], s[2], s[3], s[4], grads[0], ks, scale);
        return {dq, dk, dv, Tensor(), Tensor()};
    }
};

Tensor natten2d_autograd(const Tensor &q, const Tensor &k, const Tensor &v, int64_t ks,
                         double scale) {
    return NattenFn<true>::apply(q, k, v, ks, scale);
}
Tensor natten1d_autograd(const Tensor &q, const Tensor &k, const Tensor &v, int64_t ks,
                         double scale) {
    return NattenFn<false>::apply(q, k, v, ks, scale);
}
Tensor natten2d_plain(const Tensor &q, const Tensor &k, const Tensor &v, int64_t ks, double scale) {
    return std::get<0>(call_fwd(true, q, k, v, ks, scale));
}
Tensor natten1d_plain(const Tensor &q, const Tensor &k, const Tensor &v, int64_t ks, double scale) {
    return std::get<0>(call_fwd(false, q, k, v, ks, scale));
}

}  // namespace

TORCH_LIBRARY(enatten, m) {
    m.def("na2d_fwd(Tensor q, Tensor k, Tensor v, int kernel_size, float scale) -> (Tensor, Tensor)");
    m.def("na2d_bwd(Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, Tensor d_o, "
          "int kernel_size, float scale) -> (Tensor, Tensor, Tensor)");
    m.def("na1d_fwd(Tensor q, Tensor k, Tensor v, int kernel_size, float scale) -> (Tensor, Tensor)");
    m.def("na1d_bwd(Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, Tensor d_o, "
          "int kernel_size, float scale) -> (Tensor, Tensor, Tensor)");
    m.def("natten2d(Tensor q, Tensor k, Tensor v, int kernel_size=7, float scale=1.0) -> Tensor");
    m.def("natten1d(Tensor q, Tensor k, Tensor v, int kernel_size=7, float scale=1.0) -> Tensor");
}

TORCH_LIBRARY_IMPL(enatten, CompositeExplicitAutograd, m) {
    m.impl("na2d_fwd", &na2d_fwd);
    m.impl("na2d_bwd", &na2d_bwd);
    m.impl("na1d_fwd", &na1d_fwd);
    m.impl("na1d_bwd", &na1d_bwd);
    m.impl("natten2d", &natten2d_plain);
    m.impl("natten1d", &natten1d_plain);
}

TORCH_LIBRARY_IMPL(enatten, Autograd, m) {
    m.impl("natten2d", &natten2d_autograd);
    m.impl("natten1d", &natten1d_autograd);
}
