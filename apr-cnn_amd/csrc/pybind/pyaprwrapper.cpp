// pybind11 module with the names the reference registers on `_pyaprwrapper.aprnet` (wrappers/pythonBind.cpp:144-182):
//   aprnet.cuda      conv333_forward / _backward, conv111_forward / _backward, restrict_kernel333_forward / _backward,
//                    maxpool_forward_cuda / maxpool_backward_cuda, upsample_const_forward / _backward,
//                    reconstruct_forward / _backward, sample_particles_forward / _backward
//   aprnet.conv      convolve{111,333,133,555,155}_{forward,backward}, restrict_kernel{333,133,555,155}_{forward,backward}
//   aprnet.pool      maxpool_forward / maxpool_backward          aprnet.upsample  upsample_const_forward / _backward
//   aprnet.utils     number_particles, number_parts, number_particles_after_pooling / _after_upsampling
// Same argument order, batch loop, output allocation inside the call and exception types as the reference's wrappers
// (wrap_conv_gpu.hpp:32-133, wrap_maxpool_gpu.hpp, wrap_upsample_const_gpu.hpp, wrap_reconstruct_gpu.hpp,
// wrap_sample_particles_gpu.hpp, wrap_conv.hpp:12-49, wrap_pool.hpp:11-16, wrap_upsample.hpp:11-16), on top of the
// C ABI of libaprnet_hip.so.  Differences that follow from the boundary: `aprs` is any Python sequence of objects
// with a `plan(device_index)` method that returns the address of an aprnet_plan (pyapr.APR; the reference binds
// std::vector<APR*>), all tensors live on the GPU in both flavours (there is no CPU arithmetic behind this module),
// and kernels are enqueued on the current stream without a device synchronisation.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/aprnet_hip.h"

namespace py = pybind11;
using torch::Tensor;

namespace {

#define CHECK_CUDA(x) TORCH_CHECK(x.device().is_cuda(), #x " must be a CUDA tensor")
#define CHECK_CONTIGUOUS(x) TORCH_CHECK(x.is_contiguous(), #x " must be contiguous")
#define CHECK_INPUT(x) CHECK_CUDA(x); CHECK_CONTIGUOUS(x)           /* cuda/src/common.hpp:14-16 */

void check(int rc) {
    if (rc == 0) return;
    const std::string msg = aprnet_last_error();
    if (rc == APRNET_ERR_INVALID_ARGUMENT) throw std::invalid_argument(msg);       // -> ValueError, as std::invalid_argument does
    throw std::runtime_error(msg);                                                  // -> RuntimeError, as TORCH_CHECK does
}

std::vector<const aprnet_plan*> plans_of(const py::sequence& aprs, const Tensor& on) {
    std::vector<const aprnet_plan*> out;
    const int dev = on.device().index();
    for (const py::handle& h : aprs) {
        py::object v = h.attr("plan")(dev).attr("value");
        if (v.is_none()) throw std::runtime_error("APR has no device plan");
        out.push_back(reinterpret_cast<const aprnet_plan*>(v.cast<uintptr_t>()));
    }
    return out;
}

// one batch item per APR (the reference indexes input[b] for every APR of the list, wrap_conv_gpu.hpp:23-28): a shorter
// batch is refused here rather than read out of range
void check_batch(const std::vector<const aprnet_plan*>& plans, const Tensor& t) {
    if (t.dim() < 1 || (size_t)t.size(0) != plans.size())
        throw std::invalid_argument("the batch dimension of the tensors must equal the number of APRs");
}

std::vector<int> deltas_of(const Tensor& level_delta, size_t n) {
    TORCH_CHECK(level_delta.device().is_cpu() && level_delta.scalar_type() == torch::kInt32 && level_delta.dim() == 1,
                "level_delta must be a 1-D int32 CPU tensor");
    if ((size_t)level_delta.size(0) < n) throw std::invalid_argument("level_deltas must hold one entry per APR");
    auto acc = level_delta.accessor<int, 1>();
    std::vector<int> d(n);
    for (size_t i = 0; i < n; ++i) d[i] = acc[i];
    return d;
}

// PyTorch-ROCm presents the HIP device as "cuda": its current stream is the HIP stream under the masquerading wrapper
void* stream_of(const Tensor& t) { return (void*)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream(); }

int64_t max_over(const std::vector<const aprnet_plan*>& plans, const std::vector<int>& d, int shift, bool tree) {
    int64_t m = 0;
    for (size_t i = 0; i < plans.size(); ++i)
        m = std::max<int64_t>(m, tree ? aprnet_tree_parts(plans[i], d[i] + shift) : aprnet_number_parts(plans[i], d[i] + shift));
    return m;
}

bool is_f32(const Tensor& t) {
    if (t.scalar_type() == torch::kFloat32) return true;
    if (t.scalar_type() == torch::kFloat64) return false;
    throw std::runtime_error("aprnet operators take float32 or float64 tensors");
}

// ------------------------------------------------------------------------------------------- convolution
// weights in the device layout [S, Cout, Cin, kz, kx, ky]
Tensor conv_forward_impl(const py::sequence& aprs, Tensor input, Tensor weights, Tensor level_delta) {
    CHECK_INPUT(input); CHECK_INPUT(weights);
    if (input.size(1) != weights.size(2)) throw std::invalid_argument("convolve: input tensor shape does not match weights tensor!");
    TORCH_CHECK(input.scalar_type() == weights.scalar_type(), "weights must have the dtype of the input");
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    const int kz = weights.size(3), kx = weights.size(4), ky = weights.size(5);
    const int64_t B = input.size(0), Cin = input.size(1), N = input.size(2), Cout = weights.size(1), S = weights.size(0);
    auto output = torch::zeros({B, Cout, N}, input.options());
    void* st = stream_of(input);
    const bool f32 = is_f32(input);
    if (kz == 1 && kx == 1 && ky == 1) {
        for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
            check(f32 ? aprnet_conv111_fwd_f32(plans[b], d[b], input[b].data_ptr<float>(), N, Cin, weights.data_ptr<float>(), S, Cout, nullptr,
                                               output[b].data_ptr<float>(), N, st)
                      : aprnet_conv111_fwd_f64(plans[b], d[b], input[b].data_ptr<double>(), N, Cin, weights.data_ptr<double>(), S, Cout, nullptr,
                                               output[b].data_ptr<double>(), N, st));
        return output;
    }
    const int64_t ldt = std::max<int64_t>(max_over(plans, d, 0, true), 1);
    auto tree_data = torch::empty({Cin, ldt}, input.options());
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(f32 ? aprnet_conv_fwd_f32(plans[b], d[b], kz, kx, ky, input[b].data_ptr<float>(), N, Cin, weights.data_ptr<float>(), S, Cout,
                                        nullptr, output[b].data_ptr<float>(), N, tree_data.data_ptr<float>(), ldt, st)
                  : aprnet_conv_fwd_f64(plans[b], d[b], kz, kx, ky, input[b].data_ptr<double>(), N, Cin, weights.data_ptr<double>(), S, Cout,
                                        nullptr, output[b].data_ptr<double>(), N, tree_data.data_ptr<double>(), ldt, st));
    return output;
}

std::vector<Tensor> conv_backward_impl(const py::sequence& aprs, Tensor input, Tensor weights, Tensor grad_output, Tensor level_delta) {
    CHECK_INPUT(input); CHECK_INPUT(weights); CHECK_INPUT(grad_output);
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    const int kz = weights.size(3), kx = weights.size(4), ky = weights.size(5);
    const int64_t Cin = input.size(1), N = input.size(2), Cout = weights.size(1), S = weights.size(0), Ng = grad_output.size(2);
    auto grad_input = torch::zeros_like(input);
    auto grad_weights = torch::zeros_like(weights);
    void* st = stream_of(input);
    const bool f32 = is_f32(input);
    if (kz == 1 && kx == 1 && ky == 1) {
        for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
            check(f32 ? aprnet_conv111_bwd_f32(plans[b], d[b], input[b].data_ptr<float>(), N, Cin, weights.data_ptr<float>(), S, Cout,
                                               grad_output[b].data_ptr<float>(), Ng, grad_input[b].data_ptr<float>(), N,
                                               grad_weights.data_ptr<float>(), st)
                      : aprnet_conv111_bwd_f64(plans[b], d[b], input[b].data_ptr<double>(), N, Cin, weights.data_ptr<double>(), S, Cout,
                                               grad_output[b].data_ptr<double>(), Ng, grad_input[b].data_ptr<double>(), N,
                                               grad_weights.data_ptr<double>(), st));
        return {grad_input, grad_weights};
    }
    const int64_t ldt = std::max<int64_t>(max_over(plans, d, 0, true), 1);
    auto tree_data = torch::empty({Cin, ldt}, input.options());
    auto grad_tree = torch::empty({Cin, ldt}, input.options());
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(f32 ? aprnet_conv_bwd_f32(plans[b], d[b], kz, kx, ky, input[b].data_ptr<float>(), N, Cin, weights.data_ptr<float>(), S, Cout,
                                        grad_output[b].data_ptr<float>(), Ng, grad_input[b].data_ptr<float>(), N, grad_weights.data_ptr<float>(),
                                        tree_data.data_ptr<float>(), ldt, grad_tree.data_ptr<float>(), ldt, st)
                  : aprnet_conv_bwd_f64(plans[b], d[b], kz, kx, ky, input[b].data_ptr<double>(), N, Cin, weights.data_ptr<double>(), S, Cout,
                                        grad_output[b].data_ptr<double>(), Ng, grad_input[b].data_ptr<double>(), N, grad_weights.data_ptr<double>(),
                                        tree_data.data_ptr<double>(), ldt, grad_tree.data_ptr<double>(), ldt, st));
    return {grad_input, grad_weights};
}

void expect_stencil(const Tensor& weights, int kz, int kx, int ky, const char* who) {
    TORCH_CHECK(weights.dim() == 6 && weights.size(3) == kz && weights.size(4) == kx && weights.size(5) == ky, who,
                ": weights of another stencil size given");
}

// restrict kernel in the device layout: [S, Cout, Cin, k] -> [n_other, Cout, Cin, k]
Tensor restrict_impl(Tensor w, int64_t n_other, bool backward) {
    CHECK_INPUT(w);
    c10::DeviceGuard guard(w.device());
    auto out = torch::empty({n_other, w.size(1), w.size(2), w.size(3), w.size(4), w.size(5)}, w.options());
    const int F = w.size(1) * w.size(2), kz = w.size(3), kx = w.size(4), ky = w.size(5), S = w.size(0);
    void* st = stream_of(w);
    if (is_f32(w))
        check(backward ? aprnet_restrict_kernel_bwd_f32(w.data_ptr<float>(), S, F, kz, kx, ky, n_other, out.data_ptr<float>(), st)
                       : aprnet_restrict_kernel_fwd_f32(w.data_ptr<float>(), S, F, kz, kx, ky, n_other, out.data_ptr<float>(), st));
    else
        check(backward ? aprnet_restrict_kernel_bwd_f64(w.data_ptr<double>(), S, F, kz, kx, ky, n_other, out.data_ptr<double>(), st)
                       : aprnet_restrict_kernel_fwd_f64(w.data_ptr<double>(), S, F, kz, kx, ky, n_other, out.data_ptr<double>(), st));
    return out;
}

// CPU-flavour weight layout [Cin, S, Cout, k] (conv.py:164) <-> device layout [S, Cout, Cin, k]
Tensor to_device_layout(const Tensor& w) { return w.permute({1, 2, 0, 3, 4, 5}).contiguous(); }
Tensor to_cpu_layout(const Tensor& w) { return w.permute({2, 0, 1, 3, 4, 5}).contiguous(); }

// ------------------------------------------------------------------------------------------- pool / upsample
std::vector<Tensor> maxpool_forward_impl(const py::sequence& aprs, Tensor input, Tensor level_delta, double pad) {
    CHECK_INPUT(input);
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    const int64_t B = input.size(0), C = input.size(1), N = input.size(2), n_out = max_over(plans, d, 1, false);
    auto output = torch::full({B, C, n_out}, pad, input.options());       // maxpool.hpp:51 / wrap_maxpool_gpu.hpp:42
    auto idx = torch::zeros({B, C, n_out}, input.options().dtype(torch::kInt64));
    void* st = stream_of(input);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(input) ? aprnet_maxpool_fwd_f32(plans[b], d[b], input[b].data_ptr<float>(), N, C, output[b].data_ptr<float>(), n_out,
                                                     idx[b].data_ptr<int64_t>(), n_out, st)
                            : aprnet_maxpool_fwd_f64(plans[b], d[b], input[b].data_ptr<double>(), N, C, output[b].data_ptr<double>(), n_out,
                                                     idx[b].data_ptr<int64_t>(), n_out, st));
    return {output, idx};
}

Tensor maxpool_backward_impl(const py::sequence& aprs, Tensor grad_output, Tensor max_indices, Tensor level_delta) {
    CHECK_INPUT(grad_output); CHECK_INPUT(max_indices);
    c10::DeviceGuard guard(grad_output.device());
    auto plans = plans_of(aprs, grad_output);
    check_batch(plans, grad_output);
    auto d = deltas_of(level_delta, plans.size());
    const int64_t B = grad_output.size(0), C = grad_output.size(1), n_out = grad_output.size(2), n_in = max_over(plans, d, 0, false);
    auto grad_input = torch::zeros({B, C, n_in}, grad_output.options());
    void* st = stream_of(grad_output);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(grad_output) ? aprnet_maxpool_bwd_f32(plans[b], d[b], grad_output[b].data_ptr<float>(), n_out, C, grad_input[b].data_ptr<float>(),
                                                           n_in, max_indices[b].data_ptr<int64_t>(), max_indices.size(2), st)
                                  : aprnet_maxpool_bwd_f64(plans[b], d[b], grad_output[b].data_ptr<double>(), n_out, C,
                                                           grad_input[b].data_ptr<double>(), n_in, max_indices[b].data_ptr<int64_t>(),
                                                           max_indices.size(2), st));
    return grad_input;
}

Tensor upsample_forward_impl(const py::sequence& aprs, Tensor input, Tensor level_delta) {
    CHECK_INPUT(input);
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    for (int v : d)
        if (v <= 0)      // upsample.hpp:49-54
            throw std::invalid_argument("UpSampleConst is only implemented for downsampled particles. It is currently not possible to go "
                                        "beyond the original resolution. That is, input must have `level_delta > 0`.");
    const int64_t B = input.size(0), C = input.size(1), N = input.size(2), n_out = max_over(plans, d, -1, false);
    auto output = torch::zeros({B, C, n_out}, input.options());
    void* st = stream_of(input);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(input) ? aprnet_upsample_fwd_f32(plans[b], d[b], input[b].data_ptr<float>(), N, C, output[b].data_ptr<float>(), n_out, st)
                            : aprnet_upsample_fwd_f64(plans[b], d[b], input[b].data_ptr<double>(), N, C, output[b].data_ptr<double>(), n_out, st));
    return output;
}

Tensor upsample_backward_impl(const py::sequence& aprs, Tensor grad_output, Tensor level_delta) {
    CHECK_INPUT(grad_output);
    c10::DeviceGuard guard(grad_output.device());
    auto plans = plans_of(aprs, grad_output);
    check_batch(plans, grad_output);
    auto d = deltas_of(level_delta, plans.size());
    const int64_t B = grad_output.size(0), C = grad_output.size(1), n_out = grad_output.size(2), n_in = max_over(plans, d, 0, false);
    auto grad_input = torch::zeros({B, C, n_in}, grad_output.options());
    void* st = stream_of(grad_output);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(grad_output) ? aprnet_upsample_bwd_f32(plans[b], d[b], grad_output[b].data_ptr<float>(), n_out, C, grad_input[b].data_ptr<float>(), n_in, st)
                                  : aprnet_upsample_bwd_f64(plans[b], d[b], grad_output[b].data_ptr<double>(), n_out, C, grad_input[b].data_ptr<double>(), n_in, st));
    return grad_input;
}

// ------------------------------------------------------------------------------------------- pixels <-> particles
// dense shape of a batch at its level deltas: every item must agree (wrap_reconstruct_gpu.hpp:30-63 takes the first)
std::vector<int64_t> dense_shape(const py::sequence& aprs, const std::vector<int>& d) {
    std::vector<int64_t> shape;
    size_t i = 0;
    for (const py::handle& h : aprs) {
        const int lc = h.attr("level_max")().cast<int>() - d[i++];
        std::vector<int64_t> s = {h.attr("z_num")(lc).cast<int64_t>(), h.attr("x_num")(lc).cast<int64_t>(), h.attr("y_num")(lc).cast<int64_t>()};
        if (shape.empty()) shape = s;
        else if (shape != s) throw std::invalid_argument("reconstruct / sample_particles: all batch items must share the dense shape at their level delta");
    }
    return shape;
}

Tensor reconstruct_forward_impl(const py::sequence& aprs, Tensor input, Tensor level_delta) {
    CHECK_INPUT(input);
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    auto shape = dense_shape(aprs, d);
    const int64_t B = input.size(0), C = input.size(1), N = input.size(2), plane = shape[0] * shape[1] * shape[2];
    auto output = torch::zeros({B, C, shape[0], shape[1], shape[2]}, input.options());
    void* st = stream_of(input);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(input) ? aprnet_reconstruct_fwd_f32(plans[b], d[b], input[b].data_ptr<float>(), N, C, output[b].data_ptr<float>(), plane, st)
                            : aprnet_reconstruct_fwd_f64(plans[b], d[b], input[b].data_ptr<double>(), N, C, output[b].data_ptr<double>(), plane, st));
    return output;
}

Tensor reconstruct_backward_impl(const py::sequence& aprs, Tensor grad_output, Tensor level_delta) {
    CHECK_INPUT(grad_output);
    c10::DeviceGuard guard(grad_output.device());
    auto plans = plans_of(aprs, grad_output);
    check_batch(plans, grad_output);
    auto d = deltas_of(level_delta, plans.size());
    (void)dense_shape(aprs, d);
    const int64_t B = grad_output.size(0), C = grad_output.size(1), n = max_over(plans, d, 0, false);
    const int64_t plane = grad_output.size(2) * grad_output.size(3) * grad_output.size(4);
    auto grad_input = torch::zeros({B, C, n}, grad_output.options());
    void* st = stream_of(grad_output);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(grad_output) ? aprnet_reconstruct_bwd_f32(plans[b], d[b], grad_output[b].data_ptr<float>(), plane, C, grad_input[b].data_ptr<float>(), n, st)
                                  : aprnet_reconstruct_bwd_f64(plans[b], d[b], grad_output[b].data_ptr<double>(), plane, C, grad_input[b].data_ptr<double>(), n, st));
    return grad_input;
}

Tensor sample_forward_impl(const py::sequence& aprs, Tensor input, Tensor level_delta) {
    CHECK_INPUT(input);
    c10::DeviceGuard guard(input.device());
    auto plans = plans_of(aprs, input);
    check_batch(plans, input);
    auto d = deltas_of(level_delta, plans.size());
    (void)dense_shape(aprs, d);
    const int64_t B = input.size(0), C = input.size(1), n = max_over(plans, d, 0, false), plane = input.size(2) * input.size(3) * input.size(4);
    auto output = torch::zeros({B, C, n}, input.options());
    void* st = stream_of(input);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(input) ? aprnet_sample_particles_fwd_f32(plans[b], d[b], input[b].data_ptr<float>(), plane, C, output[b].data_ptr<float>(), n, st)
                            : aprnet_sample_particles_fwd_f64(plans[b], d[b], input[b].data_ptr<double>(), plane, C, output[b].data_ptr<double>(), n, st));
    return output;
}

Tensor sample_backward_impl(const py::sequence& aprs, Tensor grad_output, Tensor level_delta) {
    CHECK_INPUT(grad_output);
    c10::DeviceGuard guard(grad_output.device());
    auto plans = plans_of(aprs, grad_output);
    check_batch(plans, grad_output);
    auto d = deltas_of(level_delta, plans.size());
    auto shape = dense_shape(aprs, d);
    const int64_t B = grad_output.size(0), C = grad_output.size(1), N = grad_output.size(2), plane = shape[0] * shape[1] * shape[2];
    auto grad_input = torch::zeros({B, C, shape[0], shape[1], shape[2]}, grad_output.options());
    void* st = stream_of(grad_output);
    for (int64_t b = 0; b < (int64_t)plans.size(); ++b)
        check(is_f32(grad_output) ? aprnet_sample_particles_bwd_f32(plans[b], d[b], grad_output[b].data_ptr<float>(), N, C, grad_input[b].data_ptr<float>(), plane, st)
                                  : aprnet_sample_particles_bwd_f64(plans[b], d[b], grad_output[b].data_ptr<double>(), N, C, grad_input[b].data_ptr<double>(), plane, st));
    return grad_input;
}

// helpers::number_parts (helpers.hpp:86-101): host arithmetic on the row tables, no device needed
int64_t number_parts(const py::object& apr, int level_delta) {
    py::object it = apr.attr("iterator")(), tr = apr.attr("tree_iterator")();
    const int lc = apr.attr("level_max")().cast<int>() - level_delta;
    int64_t n = it.attr("particles_level_end")(lc).cast<int64_t>();
    if (lc >= tr.attr("level_min")().cast<int>() && lc <= tr.attr("level_max")().cast<int>())
        n += tr.attr("particles_level_end")(lc).cast<int64_t>() - tr.attr("particles_level_begin")(lc).cast<int64_t>();
    return n;
}

template <int KZ, int KX, int KY>
void bind_convolution(py::module& m) {
    using namespace pybind11::literals;
    const std::string name = "convolve" + std::to_string(KZ) + std::to_string(KX) + std::to_string(KY);
    m.def((name + "_forward").c_str(), [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor level_deltas) {
        expect_stencil(weights, KZ, KX, KY, "convolve_forward");
        return conv_forward_impl(aprs, input, to_device_layout(weights), level_deltas);
    }, "aprs"_a, "input"_a, "weights"_a, "level_deltas"_a);
    m.def((name + "_backward").c_str(), [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor grad_output, Tensor level_deltas) {
        expect_stencil(weights, KZ, KX, KY, "convolve_backward");
        auto g = conv_backward_impl(aprs, input, to_device_layout(weights), grad_output, level_deltas);
        return std::vector<Tensor>{g[0], to_cpu_layout(g[1])};
    }, "aprs"_a, "input"_a, "weights"_a, "grad_output"_a, "level_deltas"_a);
}

template <int KZ, int KX, int KY>
void bind_restrict(py::module& m) {
    using namespace pybind11::literals;
    const std::string name = "restrict_kernel" + std::to_string(KZ) + std::to_string(KX) + std::to_string(KY);
    m.def((name + "_forward").c_str(), [](Tensor weights, int64_t num_levels) {
        expect_stencil(weights, KZ, KX, KY, "restrict_kernel_forward");
        return to_cpu_layout(restrict_impl(to_device_layout(weights), num_levels, false));
    }, "weights"_a, "num_levels"_a);
    m.def((name + "_backward").c_str(), [](Tensor grad_weights, int64_t num_stencils) {
        expect_stencil(grad_weights, KZ, KX, KY, "restrict_kernel_backward");
        return to_cpu_layout(restrict_impl(to_device_layout(grad_weights), num_stencils, true));
    }, "grad_weights"_a, "num_stencils"_a);
}

}  // namespace

PYBIND11_MODULE(_pyaprwrapper, m) {
    using namespace pybind11::literals;
    m.doc() = "reference-named native functions of pyapr.aprnet on top of libaprnet_hip.so";
    py::module aprnet = m.def_submodule("aprnet");

    py::module utils_module = aprnet.def_submodule("utils");
    utils_module.def("number_particles", &number_parts, "apr"_a, "level_delta"_a);
    utils_module.def("number_parts", &number_parts, "apr"_a, "level_delta"_a);
    utils_module.def("number_particles_after_pooling", [](const py::object& apr, int d) { return number_parts(apr, d + 1); }, "apr"_a, "level_delta"_a);
    utils_module.def("number_particles_after_upsampling", [](const py::object& apr, int d) { return number_parts(apr, d - 1); }, "apr"_a, "level_delta"_a);

    py::module conv_module = aprnet.def_submodule("conv");
    bind_convolution<1, 1, 1>(conv_module);
    bind_convolution<3, 3, 3>(conv_module);
    bind_convolution<1, 3, 3>(conv_module);
    bind_convolution<5, 5, 5>(conv_module);
    bind_convolution<1, 5, 5>(conv_module);
    bind_restrict<3, 3, 3>(conv_module);
    bind_restrict<1, 3, 3>(conv_module);
    bind_restrict<5, 5, 5>(conv_module);
    bind_restrict<1, 5, 5>(conv_module);

    py::module pool_module = aprnet.def_submodule("pool");
    pool_module.def("maxpool_forward", [](const py::sequence& aprs, Tensor input, Tensor level_delta) {
        return maxpool_forward_impl(aprs, input, level_delta, -1e17); }, "aprs"_a, "input"_a, "level_delta"_a);
    pool_module.def("maxpool_backward", &maxpool_backward_impl, "aprs"_a, "grad_output"_a, "max_indices"_a, "level_delta"_a);

    py::module upsample_module = aprnet.def_submodule("upsample");
    upsample_module.def("upsample_const_forward", &upsample_forward_impl, "aprs"_a, "input"_a, "level_delta"_a);
    upsample_module.def("upsample_const_backward", &upsample_backward_impl, "aprs"_a, "grad_output"_a, "level_delta"_a);

    py::module cuda_module = aprnet.def_submodule("cuda");
    cuda_module.def("maxpool_forward_cuda", [](const py::sequence& aprs, Tensor input, Tensor level_delta) {
        return maxpool_forward_impl(aprs, input, level_delta, 0.0); }, "aprs"_a, "input"_a, "level_delta"_a);
    cuda_module.def("maxpool_backward_cuda", &maxpool_backward_impl, "aprs"_a, "grad_output"_a, "max_indices"_a, "level_delta"_a);
    cuda_module.def("conv111_forward", [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor level_delta) {
        expect_stencil(weights, 1, 1, 1, "conv111_forward");
        return conv_forward_impl(aprs, input, weights, level_delta); }, "aprs"_a, "input"_a, "weights"_a, "level_delta"_a);
    cuda_module.def("conv111_backward", [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor grad_output, Tensor level_delta) {
        expect_stencil(weights, 1, 1, 1, "conv111_backward");
        return conv_backward_impl(aprs, input, weights, grad_output, level_delta); },
        "aprs"_a, "input"_a, "weights"_a, "grad_output"_a, "level_delta"_a);
    cuda_module.def("conv333_forward", [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor level_delta) {
        expect_stencil(weights, 3, 3, 3, "conv333_forward");
        return conv_forward_impl(aprs, input, weights, level_delta); }, "aprs"_a, "input"_a, "weights"_a, "level_delta"_a);
    cuda_module.def("conv333_backward", [](const py::sequence& aprs, Tensor input, Tensor weights, Tensor grad_output, Tensor level_delta) {
        expect_stencil(weights, 3, 3, 3, "conv333_backward");
        return conv_backward_impl(aprs, input, weights, grad_output, level_delta); },
        "aprs"_a, "input"_a, "weights"_a, "grad_output"_a, "level_delta"_a);
    cuda_module.def("upsample_const_forward", &upsample_forward_impl, "aprs"_a, "input"_a, "level_delta"_a);
    cuda_module.def("upsample_const_backward", &upsample_backward_impl, "aprs"_a, "grad_output"_a, "level_delta"_a);
    cuda_module.def("restrict_kernel333_forward", [](Tensor weights, int64_t num_levels) {
        expect_stencil(weights, 3, 3, 3, "restrict_kernel333_forward");
        return restrict_impl(weights, num_levels, false); }, "weights"_a, "num_levels"_a);
    cuda_module.def("restrict_kernel333_backward", [](Tensor grad_weights_expanded, int64_t num_levels) {
        expect_stencil(grad_weights_expanded, 3, 3, 3, "restrict_kernel333_backward");
        return restrict_impl(grad_weights_expanded, num_levels, true); }, "grad_weights_expanded"_a, "num_levels"_a);
    cuda_module.def("reconstruct_forward", &reconstruct_forward_impl, "aprs"_a, "input"_a, "level_delta"_a);
    cuda_module.def("reconstruct_backward", &reconstruct_backward_impl, "aprs"_a, "grad_output"_a, "level_delta"_a);
    cuda_module.def("sample_particles_forward", &sample_forward_impl, "aprs"_a, "input"_a, "level_delta"_a);
    cuda_module.def("sample_particles_backward", &sample_backward_impl, "aprs"_a, "grad_output"_a, "level_delta"_a);
}
