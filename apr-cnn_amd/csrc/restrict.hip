// RestrictKernel<kz,kx,ky>::forward/backward (kernel.hpp:31-224): stencils of levels >= S are the
// last given stencil restricted by area overlap with step 2^(level-S+1) and divided by step^ndim
// (ndim counts the non-singleton dimensions only, kernel.hpp:59).  Tiny: one thread per filter
// element, gather form in both directions, so the result is deterministic.
#include "common.hpp"

#include <mutex>

namespace aprnet {

__device__ __forceinline__ float overlap1(int o, int i, int k, int step) {
    const int off = (k / 2) * step - k / 2;
    const int v = min((o + 1) * step, off + i + step) - max(o * step, off + i);
    return (float)max(v, 0);
}

// w [S][F][K] -> we [S_exp][F][K]
template <typename T>
__global__ void restrict_fwd_kernel(const T* __restrict__ w, T* __restrict__ we, int S, int S_exp, int F,
                                    int kz, int kx, int ky, int ndim) {
    const int K = kz * kx * ky;
    const int64_t n = (int64_t)S_exp * F * K;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const int tap = (int)(e % K);
    const int f = (int)((e / K) % F);
    const int l = (int)(e / ((int64_t)K * F));
    if (l < S) { we[e] = w[e]; return; }
    const int step = 1 << (l - (S - 1));
    const float factor = powf((float)step, (float)ndim);
    const int zo = tap / (kx * ky), xo = (tap / ky) % kx, yo = tap % ky;
    const T* src = w + ((int64_t)(S - 1) * F + f) * K;
    T acc = 0;
    // same tap order as the reference: z_in, x_in, y_in ascending
    for (int zi = 0; zi < kz; ++zi) {
        const float oz = overlap1(zo, zi, kz, step);
        if (oz <= 0) continue;
        for (int xi = 0; xi < kx; ++xi) {
            const float ox = overlap1(xo, xi, kx, step);
            if (ox <= 0) continue;
            for (int yi = 0; yi < ky; ++yi) {
                const float oy = overlap1(yo, yi, ky, step);
                if (oy <= 0) continue;
                const float ov = ox * oy * oz / factor;
                acc += (T)ov * src[(zi * kx + xi) * ky + yi];
            }
        }
    }
    we[e] = acc;
}

// gwe [S_exp][F][K] -> gw [S][F][K]
template <typename T>
__global__ void restrict_bwd_kernel(const T* __restrict__ gwe, T* __restrict__ gw, int S, int S_exp, int F,
                                    int kz, int kx, int ky, int ndim) {
    const int K = kz * kx * ky;
    const int64_t n = (int64_t)S * F * K;
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= n) return;
    const int tap = (int)(e % K);
    const int f = (int)((e / K) % F);
    const int l = (int)(e / ((int64_t)K * F));
    T acc = gwe[e];
    if (l == S - 1) {
        const int zi = tap / (kx * ky), xi = (tap / ky) % kx, yi = tap % ky;
        for (int le = S; le < S_exp; ++le) {
            const int step = 1 << (le - (S - 1));
            const float factor = powf((float)step, (float)ndim);
            const T* src = gwe + ((int64_t)le * F + f) * K;
            for (int zo = 0; zo < kz; ++zo) {
                const float oz = overlap1(zo, zi, kz, step);
                if (oz <= 0) continue;
                for (int xo = 0; xo < kx; ++xo) {
                    const float ox = overlap1(xo, xi, kx, step);
                    if (ox <= 0) continue;
                    for (int yo = 0; yo < ky; ++yo) {
                        const float oy = overlap1(yo, yi, ky, step);
                        if (oy <= 0) continue;
                        const float ov = ox * oy * oz / factor;
                        acc += (T)ov * src[(zo * kx + xo) * ky + yo];
                    }
                }
            }
        }
    }
    gw[e] = acc;
}

template <typename T, bool Backward>
int restrict_kernel(const T* src, int S, int F, int kz, int kx, int ky, int S_exp, T* dst, hipStream_t st) {
    if (S <= 0 || S_exp < S || F <= 0 || kz <= 0 || kx <= 0 || ky <= 0)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "restrict_kernel: need 0 < S <= S_exp and a non-empty filter bank");
    const int ndim = (kz > 1) + (kx > 1) + (ky > 1);
    const int64_t n = (int64_t)(Backward ? S : S_exp) * F * kz * kx * ky;
    dim3 grid((unsigned)((n + 255) / 256));
    if (!Backward) hipLaunchKernelGGL(restrict_fwd_kernel<T>, grid, dim3(256), 0, st, src, dst, S, S_exp, F, kz, kx, ky, ndim);
    else hipLaunchKernelGGL(restrict_bwd_kernel<T>, grid, dim3(256), 0, st, src, dst, S, S_exp, F, kz, kx, ky, ndim);
    APRNET_LAUNCH_CHECK("restrict_kernel");
    return 0;
}

// ---------------------------------------------------------------------------- bias gradient
// grad_bias[c] = sum over batch and positions of grad_output (conv.py:33): two passes, fixed summation
// order (no atomics), so the result is the same from run to run.
constexpr int CS_BLOCKS = 256, CS_TB = 256;

template <typename T>
__global__ void __launch_bounds__(CS_TB)
channel_sum_partial_kernel(const T* __restrict__ x, int64_t ld, int64_t n, typename Num<T>::acc* __restrict__ partial) {
    typedef typename Num<T>::acc A;
    __shared__ A red[CS_TB / 64];
    const T* row = x + (int64_t)blockIdx.y * ld;
    A s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    const int64_t stride = (int64_t)gridDim.x * CS_TB;
    int64_t i = (int64_t)blockIdx.x * CS_TB + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {
        s0 += Num<T>::ld(row[i]); s1 += Num<T>::ld(row[i + stride]);
        s2 += Num<T>::ld(row[i + 2 * stride]); s3 += Num<T>::ld(row[i + 3 * stride]);
    }
    for (; i < n; i += stride) s0 += Num<T>::ld(row[i]);
    A s = (s0 + s1) + (s2 + s3);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        A t = 0;
#pragma unroll
        for (int w = 0; w < CS_TB / 64; ++w) t += red[w];
        partial[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

template <typename T>
__global__ void __launch_bounds__(64)
channel_sum_final_kernel(const T* __restrict__ partial, int nb, T* __restrict__ out, int accumulate) {
    T s = 0;
    for (int i = threadIdx.x; i < nb; i += 64) s += partial[(int64_t)blockIdx.x * nb + i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
    if (threadIdx.x == 0) out[blockIdx.x] = accumulate ? out[blockIdx.x] + s : s;
}

template <typename T>
int channel_sum(const T* x, int64_t ld, int C, int64_t n, typename Num<T>::acc* out, int accumulate, typename Num<T>::acc* work,
                hipStream_t st) {
    if (C <= 0) return 0;
    if (!x || !out || !work || n < 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "channel_sum: null argument");
    hipLaunchKernelGGL(channel_sum_partial_kernel<T>, dim3(CS_BLOCKS, (unsigned)C), dim3(CS_TB), 0, st, x, ld, n, work);
    hipLaunchKernelGGL(channel_sum_final_kernel<typename Num<T>::acc>, dim3((unsigned)C), dim3(64), 0, st, work, CS_BLOCKS, out, accumulate);
    APRNET_LAUNCH_CHECK("channel_sum kernels");
    return 0;
}

// ---------------------------------------------------------------------------- bias gradient without a work-space argument
// The block partials of channel_sum live in a device array of this library instead of caller memory, for callers that
// cannot allocate (under stream capture, in serving loops).  Every GPU holds its own copy of the array at its own
// address; host code only ever uses the address that hipGetSymbolAddress returned on that GPU, never the array's name.
constexpr int CS_STATIC_MAX_C = 1024;
constexpr int CS_MAX_DEVICES = 64;
static __device__ __align__(256) float cs_static_scratch[CS_STATIC_MAX_C * CS_BLOCKS];     // 1 MiB per GPU
static float* g_cs_static_ptr[CS_MAX_DEVICES] = {};
static std::mutex g_cs_static_mutex;

static int cs_static_scratch_ptr(float** out) {
    int dev = -1;
    APRNET_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= CS_MAX_DEVICES) return fail(APRNET_ERR_UNSUPPORTED, "channel_sum_static: device index beyond 63");
    std::lock_guard<std::mutex> lock(g_cs_static_mutex);
    if (!g_cs_static_ptr[dev]) {
        float* ptr = nullptr;
        APRNET_HIP_CHECK(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(cs_static_scratch)));
        if (!ptr) return fail(APRNET_ERR_HIP, "channel_sum_static: the scratch array has no address on this device");
        g_cs_static_ptr[dev] = ptr;
    }
    *out = g_cs_static_ptr[dev];
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
int aprnet_channel_sum_static_max_channels(void) { return CS_STATIC_MAX_C; }
int aprnet_channel_sum_static_f32(const float* x, int64_t ld, int C, int64_t n, float* out, int accumulate, void* st) {
    if (C > CS_STATIC_MAX_C)
        return fail(APRNET_ERR_UNSUPPORTED, "channel_sum_static: at most " + std::to_string(CS_STATIC_MAX_C) +
                                            " channels per call (" + std::to_string(C) + " given); use aprnet_channel_sum_f32 with a work space");
    if (C <= 0) return 0;
    float* work = nullptr;
    if (int rc = cs_static_scratch_ptr(&work)) return rc;
    // the partial kernel writes every slot it later reads (C * CS_BLOCKS values): nothing of an earlier call survives
    return channel_sum<float>(x, ld, C, n, out, accumulate, work, (hipStream_t)st);
}
int aprnet_channel_sum_work_elems(int C) { return C * CS_BLOCKS; }
int aprnet_channel_sum_f32(const float* x, int64_t ld, int C, int64_t n, float* out, int accumulate, float* work, void* st) {
    return channel_sum<float>(x, ld, C, n, out, accumulate, work, (hipStream_t)st);
}
int aprnet_channel_sum_bf16(const uint16_t* x, int64_t ld, int C, int64_t n, float* out, int accumulate, float* work, void* st) {
    return channel_sum<bf16_t>((const bf16_t*)x, ld, C, n, out, accumulate, work, (hipStream_t)st);
}
int aprnet_channel_sum_f64(const double* x, int64_t ld, int C, int64_t n, double* out, int accumulate, double* work, void* st) {
    return channel_sum<double>(x, ld, C, n, out, accumulate, work, (hipStream_t)st);
}
#define RESTRICT_API(T, SFX)                                                                                           \
    int aprnet_restrict_kernel_fwd_##SFX(const T* w, int S, int F, int kz, int kx, int ky, int S_exp, T* we, void* st) { \
        return restrict_kernel<T, false>(w, S, F, kz, kx, ky, S_exp, we, (hipStream_t)st); }                           \
    int aprnet_restrict_kernel_bwd_##SFX(const T* gwe, int S_exp, int F, int kz, int kx, int ky, int S, T* gw, void* st) { \
        return restrict_kernel<T, true>(gwe, S, F, kz, kx, ky, S_exp, gw, (hipStream_t)st); }
RESTRICT_API(float, f32)
RESTRICT_API(double, f64)
}
