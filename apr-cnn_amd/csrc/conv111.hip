// 1x1x1 convolution: Convolution<1,1,1>::forward/backward (conv.hpp:199-256, 484-554).
// Particles of one level are contiguous in the feature vector (conv111_gpu.cu:30-31), and so are the
// downsampled particles, so the operator is a per-segment channel GEMM: out[co][i] = sum_ci w[s][co][ci] x[ci][i]
// with the stencil index s = min(S-1, Lc-level) constant per segment.  One launch per segment keeps
// the weights wave-uniform (scalar loads); x is read once per block of COB output channels.
#include "common.hpp"

namespace aprnet {

constexpr int TB1 = 256;

// dst[o][i] = sum_c W(o, c) * src[c][i],  W(o, c) = w[o * so + c * sc]
template <typename T, int OB>
__global__ void __launch_bounds__(TB1)
conv111_kernel(const T* __restrict__ src, int64_t lds, int Csrc, const T* __restrict__ w, int so, int sc,
               const T* __restrict__ bias, T* __restrict__ dst, int64_t ldd, int Cdst, int64_t begin, int64_t end) {
    const int64_t i = begin + (int64_t)blockIdx.x * TB1 + threadIdx.x;
    if (i >= end) return;
    const int o0 = blockIdx.y * OB;
    T acc[OB];
#pragma unroll
    for (int o = 0; o < OB; ++o) acc[o] = 0;
    for (int c = 0; c < Csrc; ++c) {
        const T v = src[(int64_t)c * lds + i];
#pragma unroll
        for (int o = 0; o < OB; ++o)
            if (o0 + o < Cdst) acc[o] += w[(int64_t)(o0 + o) * so + (int64_t)c * sc] * v;
    }
#pragma unroll
    for (int o = 0; o < OB; ++o)
        if (o0 + o < Cdst) dst[(int64_t)(o0 + o) * ldd + i] = acc[o] + (bias ? bias[o0 + o] : (T)0);
}

// gw[co][ci] += sum_i gy[co][i] * x[ci][i] over [begin, end): 8x8 register tile per thread, block
// reduction through LDS, one atomic per (co, ci) and block.
template <typename T>
__global__ void __launch_bounds__(TB1)
conv111_dw_kernel(const T* __restrict__ x, int64_t ldx, int Cin, const T* __restrict__ gy, int64_t ldy, int Cout,
                  T* __restrict__ gw, int64_t begin, int64_t end) {
    constexpr int B = 8;
    __shared__ T red[TB1 / 64][B * B];
    const int co0 = blockIdx.y * B, ci0 = blockIdx.z * B;
    T acc[B][B];
#pragma unroll
    for (int a = 0; a < B; ++a)
#pragma unroll
        for (int b = 0; b < B; ++b) acc[a][b] = 0;
    for (int64_t i = begin + (int64_t)blockIdx.x * TB1 + threadIdx.x; i < end; i += (int64_t)gridDim.x * TB1) {
        T g[B], v[B];
#pragma unroll
        for (int a = 0; a < B; ++a) g[a] = co0 + a < Cout ? gy[(int64_t)(co0 + a) * ldy + i] : (T)0;
#pragma unroll
        for (int b = 0; b < B; ++b) v[b] = ci0 + b < Cin ? x[(int64_t)(ci0 + b) * ldx + i] : (T)0;
#pragma unroll
        for (int a = 0; a < B; ++a)
#pragma unroll
            for (int b = 0; b < B; ++b) acc[a][b] += g[a] * v[b];
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int a = 0; a < B; ++a)
#pragma unroll
        for (int b = 0; b < B; ++b) {
            T s = acc[a][b];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
            if (lane == 0) red[wave][a * B + b] = s;
        }
    __syncthreads();
    if (threadIdx.x < B * B) {
        T s = 0;
#pragma unroll
        for (int wv = 0; wv < TB1 / 64; ++wv) s += red[wv][threadIdx.x];
        const int a = threadIdx.x / B, b = threadIdx.x % B;
        if (co0 + a < Cout && ci0 + b < Cin) atomicAdd(&gw[(int64_t)(co0 + a) * Cin + (ci0 + b)], s);
    }
}

struct Segment { int64_t begin, end; int stencil; };

static std::vector<Segment> segments(const aprnet_plan* p, int d, int S) {
    std::vector<Segment> segs;
    const int Lc = p->lc(d);
    for (int l = Lc; l >= p->apr.level_min; --l) {
        const int s = std::min(S - 1, Lc - l);
        if (p->apr.level_end(l) > p->apr.level_begin(l)) segs.push_back({p->apr.level_begin(l), p->apr.level_end(l), s});
        if (l == Lc && Lc < p->apr.level_max) {
            const int64_t off = p->tree_offset(Lc);
            if (p->tree.level_end(Lc) > p->tree.level_begin(Lc))
                segs.push_back({p->tree.level_begin(Lc) + off, p->tree.level_end(Lc) + off, s});
        }
    }
    return segs;
}

template <typename T>
int conv111_fwd(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout,
                const T* bias, T* y, int64_t ldy, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "conv111_forward")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_forward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    constexpr int OB = 16;
    for (const Segment& sg : segments(p, d, S)) {
        dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cout + OB - 1) / OB));
        hipLaunchKernelGGL((conv111_kernel<T, OB>), grid, dim3(TB1), 0, st, x, ldx, Cin, w + (int64_t)sg.stencil * Cout * Cin,
                           Cin, 1, bias, y, ldy, Cout, sg.begin, sg.end);
    }
    APRNET_LAUNCH_CHECK("conv111_kernel");
    return 0;
}

template <typename T>
int conv111_bwd(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout, const T* gy,
                int64_t ldy, T* gx, int64_t ldgx, T* gw, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "conv111_backward")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_backward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    constexpr int OB = 16;
    for (const Segment& sg : segments(p, d, S)) {
        const T* ws = w + (int64_t)sg.stencil * Cout * Cin;
        dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cin + OB - 1) / OB));
        // grad_x[ci][i] = sum_co w[co][ci] * gy[co][i]: the same kernel with the weight strides swapped
        hipLaunchKernelGGL((conv111_kernel<T, OB>), grid, dim3(TB1), 0, st, gy, ldy, Cout, ws, 1, Cin, (const T*)nullptr, gx, ldgx, Cin,
                           sg.begin, sg.end);
        const int64_t n = sg.end - sg.begin;
        dim3 g2((unsigned)std::min<int64_t>((n + TB1 * 8 - 1) / (TB1 * 8), 256), (unsigned)((Cout + 7) / 8), (unsigned)((Cin + 7) / 8));
        hipLaunchKernelGGL(conv111_dw_kernel<T>, g2, dim3(TB1), 0, st, x, ldx, Cin, gy, ldy, Cout,
                           gw + (int64_t)sg.stencil * Cout * Cin, sg.begin, sg.end);
    }
    APRNET_LAUNCH_CHECK("conv111 backward kernels");
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
#define CONV111_API(T, SFX)                                                                                        \
    int aprnet_conv111_fwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S,  \
                                 int Cout, const T* bias, T* y, int64_t ldy, void* st) {                            \
        return conv111_fwd<T>(p, d, x, ldx, Cin, w, S, Cout, bias, y, ldy, (hipStream_t)st); }                      \
    int aprnet_conv111_bwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S,  \
                                 int Cout, const T* gy, int64_t ldy, T* gx, int64_t ldgx, T* gw, void* st) {        \
        return conv111_bwd<T>(p, d, x, ldx, Cin, w, S, Cout, gy, ldy, gx, ldgx, gw, (hipStream_t)st); }
CONV111_API(float, f32)
CONV111_API(double, f64)
}
