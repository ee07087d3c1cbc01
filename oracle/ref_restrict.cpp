// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
// Thin C driver around the reference's own RestrictKernel (pyapr/aprnet/src/kernel.hpp:10-224),
// which is compiled where it lies under /root/reference (include path given by the Makefile; the
// header is never copied).  kernel.hpp is the one header of the CPU path that depends only on
// libtorch, so it is the one piece of the reference that builds in this image; the others include
// LibAPR headers (helpers.hpp:10-11) that do not exist here.
#include <torch/all.h>
#include "kernel.hpp"

namespace {
template <int Z, int X, int Y>
void run(bool backward, const double* src, double* dst, int cin, int s_in, int s_out, int cout) {
    torch::Tensor in = torch::from_blob(const_cast<double*>(src), {cin, s_in, cout, Z, X, Y}, torch::kFloat64);
    torch::Tensor out = backward ? RestrictKernel<Z, X, Y>::backward(in, s_out) : RestrictKernel<Z, X, Y>::forward(in, s_out);
    std::memcpy(dst, out.contiguous().data_ptr<double>(), out.numel() * sizeof(double));
}
}  // namespace

// src: [cin][s_in][cout][kz][kx][ky] doubles; dst: same with s_out.  Returns 0, or -1 for an
// unsupported stencil size.
extern "C" int ref_restrict_kernel(int backward, int kz, int kx, int ky, const double* src, double* dst,
                                   int cin, int s_in, int s_out, int cout) {
    const int code = kz * 100 + kx * 10 + ky;
    switch (code) {
        case 333: run<3, 3, 3>(backward, src, dst, cin, s_in, s_out, cout); return 0;
        case 133: run<1, 3, 3>(backward, src, dst, cin, s_in, s_out, cout); return 0;
        case 155: run<1, 5, 5>(backward, src, dst, cin, s_in, s_out, cout); return 0;
        case 555: run<5, 5, 5>(backward, src, dst, cin, s_in, s_out, cout); return 0;
    }
    return -1;
}
