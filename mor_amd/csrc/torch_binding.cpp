// C++ registrations of the 14 `mor` operators for the CUDA dispatch key (which HIP tensors use under ROCm): the host
// launchers of the reference (mor/csrc/cuda/fake_quantize.cu, "FQ": fake_quantize_cuda :1839-1871, _no_alloc
// :1876-1907, quant_dequant / e4m3_with_e8_scale :1909-2011, block scaling :2013-2230, e8mx :2232-2397, channel
// scaling :2431-2660, TORCH_LIBRARY_IMPL :2663-2678) rewritten as checks + allocations + one call into the C ABI of
// libmor_hip.so.  The schemas are defined by mor_amd/ops.py; this file only provides faster implementations than
// the Python ones (a few microseconds per call instead of ~14).  It contains no kernels and no arithmetic.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <ATen/core/dispatch/Dispatcher.h>
#include <torch/csrc/autograd/custom_function.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include "../../include/mor_hip.h"

namespace {

// set through mor_torch_set_flags (mor.ops.set_flavour); per host thread, so that a thread that switches the flavour
// for a debugging session does not change the results of the others
thread_local uint32_t g_flags = MOR_FLAG_DEFAULT;

void check(int rc) { TORCH_CHECK(rc == 0, "mor_hip: ", mor_last_error()); }

void check_input(const at::Tensor& t, at::ScalarType dtype, int64_t rows, int64_t cols, const char* what) {
    TORCH_CHECK(t.scalar_type() == dtype, "mor: ", what, " must be ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(t.dim() == 2 && t.size(0) == rows && t.size(1) == cols, "mor: ", what, " must have shape (", rows, ", ", cols,
                "), got ", t.sizes());
    TORCH_CHECK(t.is_cuda(), "mor: ", what, " must be a GPU tensor");
}

void check_blocks(int64_t bx, int64_t by) { TORCH_CHECK(bx > 0 && by > 0, "mor: block dims must be positive, got (", bx, ", ", by, ")"); }

inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline void* stream_of(const at::Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

std::vector<at::Tensor> fake_quantize(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y,
                                      double clamp_threshold, int64_t mode, int64_t sf_type) {
    check_input(input, at::kBFloat16, dim_x, dim_y, "input");
    check_blocks(block_x, block_y);
    const at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor out = at::empty_like(x);
    at::Tensor meta = at::empty({cdiv(dim_x, block_x), cdiv(dim_y, block_y)}, x.options().dtype(at::kInt));
    check(mor_fake_quantize(x.data_ptr(), out.data_ptr(), meta.data_ptr<int32_t>(), dim_x, dim_y, block_x, block_y,
                            clamp_threshold, mode, sf_type, g_flags, stream_of(x)));
    return {out, meta};
}

at::Tensor fake_quantize_no_alloc(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y,
                                  double clamp_threshold, int64_t mode, int64_t sf_type, at::Tensor result) {
    check_input(input, at::kBFloat16, dim_x, dim_y, "input");
    check_input(result, at::kBFloat16, dim_x, dim_y, "result");
    TORCH_CHECK(result.is_contiguous(), "mor: result must be contiguous");
    check_blocks(block_x, block_y);
    const at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor meta = at::empty({cdiv(dim_x, block_x), cdiv(dim_y, block_y)}, x.options().dtype(at::kInt));
    check(mor_fake_quantize(x.data_ptr(), result.data_ptr(), meta.data_ptr<int32_t>(), dim_x, dim_y, block_x, block_y,
                            clamp_threshold, mode, sf_type, g_flags, stream_of(x)));
    return meta;
}

std::vector<at::Tensor> scaling(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y,
                                double e4m3_threshold, int64_t ss_mode, bool channel, bool inplace) {
    check_input(input, at::kBFloat16, dim_x, dim_y, "input");
    check_blocks(block_x, block_y);
    TORCH_CHECK(dim_x % block_x == 0 && dim_y % block_y == 0, "mor: block (", block_x, ", ", block_y,
                ") does not divide the tensor (", dim_x, ", ", dim_y, ")");
    at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor out = inplace ? x : at::empty_like(x);
    const auto i32 = x.options().dtype(at::kInt), f32 = x.options().dtype(at::kFloat);
    at::Tensor meta = at::empty({1}, i32), gamax = at::empty({1}, f32), gnnz = at::empty({1}, i32), gerr = at::empty({1}, f32);
    const size_t nbytes = mor_workspace_bytes(channel ? MOR_OP_CHANNEL_SCALING : MOR_OP_BLOCK_SCALING, dim_x, dim_y, block_x, block_y);
    at::Tensor ws = at::empty({(int64_t)nbytes}, x.options().dtype(at::kByte));
    check(mor_block_scaling(x.data_ptr(), out.data_ptr(), meta.data_ptr<int32_t>(), gamax.data_ptr<float>(), gnnz.data_ptr<int32_t>(),
                            gerr.data_ptr<float>(), dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode, channel ? 1 : 0,
                            ws.data_ptr(), nbytes, g_flags, stream_of(x)));
    if (inplace) {
        if (x.data_ptr() != input.data_ptr()) const_cast<at::Tensor&>(input).copy_(x);   // a non-contiguous input went through a copy
        return {meta, gamax, gnnz, gerr};
    }
    return {out, meta, gamax, gnnz, gerr};
}

at::Tensor e8mx_impl(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y, int64_t quantize_type,
                     int64_t scaling_strategy, const at::Tensor* result) {
    check_input(input, at::kBFloat16, dim_x, dim_y, "input");
    check_blocks(block_x, block_y);
    if (result) {
        check_input(*result, at::kBFloat16, dim_x, dim_y, "result");
        TORCH_CHECK(result->is_contiguous(), "mor: result must be contiguous");
    }
    const at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor out = result ? *result : at::empty_like(x);
    const size_t nbytes = mor_workspace_bytes(MOR_OP_E8MX, dim_x, dim_y, block_x, block_y);
    at::Tensor ws = at::empty({(int64_t)nbytes}, x.options().dtype(at::kByte));
    check(mor_e8mx(x.data_ptr(), out.data_ptr(), dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy, ws.data_ptr(), nbytes,
                   g_flags, stream_of(x)));
    return out;
}

template <int FMT>
at::Tensor quant_dequant(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t, int64_t) {
    check_input(input, at::kFloat, dim_x, dim_y, "input");
    const at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor out = at::empty_like(x);
    check(mor_quant_dequant(x.data_ptr<float>(), out.data_ptr<float>(), x.numel(), FMT, stream_of(x)));
    return out;
}

template <int RNE>
at::Tensor e8_scale(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t, int64_t) {
    check_input(input, at::kFloat, dim_x, dim_y, "input");
    const at::Tensor x = input.contiguous();
    const c10::OptionalDeviceGuard guard(x.device());
    at::Tensor out = at::empty_like(x);
    check(mor_e4m3_with_e8_scale(x.data_ptr<float>(), out.data_ptr<float>(), x.numel(), RNE, stream_of(x)));
    return out;
}

// Straight-through estimator (mor/ops.py:15-156): the gradient of the first output passes to the input unchanged.
// `call` runs the operator below the autograd key, through the dispatcher, so fake / functional tensors still trace.
using OpCall = std::function<std::vector<at::Tensor>(const at::Tensor&)>;
struct StraightThrough : public torch::autograd::Function<StraightThrough> {
    static torch::autograd::variable_list forward(torch::autograd::AutogradContext* ctx, const at::Tensor& input, OpCall call) {
        at::AutoDispatchBelowADInplaceOrView below;
        std::vector<at::Tensor> outs = call(input);
        if (outs.size() > 1) ctx->mark_non_differentiable(torch::autograd::variable_list(outs.begin() + 1, outs.end()));
        return outs;
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext*, torch::autograd::variable_list grads) {
        return {grads[0], at::Tensor()};
    }
};

std::vector<at::Tensor> fake_quantize_autograd(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y,
                                               double clamp_threshold, int64_t mode, int64_t sf_type) {
    static auto op = c10::Dispatcher::singleton().findSchemaOrThrow("mor::fake_quantize", "")
        .typed<std::vector<at::Tensor>(const at::Tensor&, int64_t, int64_t, int64_t, int64_t, double, int64_t, int64_t)>();
    return StraightThrough::apply(input, OpCall([=](const at::Tensor& x) { return op.call(x, dim_x, dim_y, block_x, block_y, clamp_threshold, mode, sf_type); }));
}

template <bool CHANNEL>
std::vector<at::Tensor> scaling_autograd(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y,
                                         double e4m3_threshold, int64_t ss_mode) {
    static auto op = c10::Dispatcher::singleton().findSchemaOrThrow(CHANNEL ? "mor::fake_quantize_channel_scaling" : "mor::fake_quantize_block_scaling", "")
        .typed<std::vector<at::Tensor>(const at::Tensor&, int64_t, int64_t, int64_t, int64_t, double, int64_t)>();
    return StraightThrough::apply(input, OpCall([=](const at::Tensor& x) { return op.call(x, dim_x, dim_y, block_x, block_y, e4m3_threshold, ss_mode); }));
}

at::Tensor e8mx_autograd(const at::Tensor& input, int64_t dim_x, int64_t dim_y, int64_t block_x, int64_t block_y, int64_t quantize_type,
                         int64_t scaling_strategy) {
    static auto op = c10::Dispatcher::singleton().findSchemaOrThrow("mor::fake_quantize_e8mx", "")
        .typed<at::Tensor(const at::Tensor&, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t)>();
    return StraightThrough::apply(input, OpCall([=](const at::Tensor& x) {
        return std::vector<at::Tensor>{op.call(x, dim_x, dim_y, block_x, block_y, quantize_type, scaling_strategy)}; }))[0];
}

}  // namespace

// mor.ops.set_flavour: MOR_FLAG_* bits for every later call of the calling thread
extern "C" __attribute__((visibility("default"))) void mor_torch_set_flags(uint32_t flags) { g_flags = flags; }

TORCH_LIBRARY_IMPL(mor, CUDA, m) {
    m.impl("fake_quantize", &fake_quantize);
    m.impl("fake_quantize_no_alloc", &fake_quantize_no_alloc);
    m.impl("quant_dequant_e4m3", &quant_dequant<MOR_FMT_E4M3>);
    m.impl("quant_dequant_e5m2", &quant_dequant<MOR_FMT_E5M2>);
    m.impl("quant_dequant_e3m2", &quant_dequant<MOR_FMT_E3M2>);
    m.impl("quant_dequant_e2m3", &quant_dequant<MOR_FMT_E2M3>);
    m.impl("e4m3_with_e8_scale_rne", &e8_scale<1>);
    m.impl("e4m3_with_e8_scale_rz", &e8_scale<0>);
    m.impl("fake_quantize_block_scaling", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, double t, int64_t s) {
        return scaling(i, x, y, bx, by, t, s, false, false); });
    m.impl("fake_quantize_block_scaling_inplace", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, double t, int64_t s) {
        return scaling(i, x, y, bx, by, t, s, false, true); });
    m.impl("fake_quantize_channel_scaling", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, double t, int64_t s) {
        return scaling(i, x, y, bx, by, t, s, true, false); });
    m.impl("fake_quantize_channel_scaling_inplace", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, double t, int64_t s) {
        return scaling(i, x, y, bx, by, t, s, true, true); });
    m.impl("fake_quantize_e8mx", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, int64_t q, int64_t s) {
        return e8mx_impl(i, x, y, bx, by, q, s, nullptr); });
    m.impl("fake_quantize_e8mx_inplace", [](const at::Tensor& i, int64_t x, int64_t y, int64_t bx, int64_t by, int64_t q, int64_t s, at::Tensor result) {
        e8mx_impl(i, x, y, bx, by, q, s, &result); });
}

// autograd for the four differentiable forward ops; the in-place / no_alloc / test ops keep their Python registration
TORCH_LIBRARY_IMPL(mor, Autograd, m) {
    m.impl("fake_quantize", &fake_quantize_autograd);
    m.impl("fake_quantize_block_scaling", &scaling_autograd<false>);
    m.impl("fake_quantize_channel_scaling", &scaling_autograd<true>);
    m.impl("fake_quantize_e8mx", &e8mx_autograd);
}
