// Normalisation over the particle axis with the ReLU that follows it: the torch.nn.BatchNorm1d / GroupNorm +
// activation of BasicBlock (apr_models/unet/unet_parts.py:17-26) on [batch, channels, particles] tensors.
//
// Both norms are "statistics over sets of rows": a row is one (batch, channel) line of the tensor; BatchNorm joins
// the rows of one channel over the batch, GroupNorm the rows of one group.  The streaming kernels work per row and
// are HBM-bound; two one-launch kernels (norm_coeffs_fwd / norm_coeffs_bwd) join the per-row results into per-set
// statistics and hand back per-row coefficients, so that a layer costs four launches each way.
//
//   forward   row_moments : mean and sum of squared deviations per row               reads x once
//             norm_apply  : y = (x - mean) * scale + shift, optional ReLU            reads x, writes y
//   backward  bwd_sums    : sum g and sum g * xhat per row, g = gy masked by y > 0   reads gy, x (, y)
//             bwd_apply   : gx = a * g + b * xhat + c                                reads gy, x (, y), writes gx
//
// Elements are moved four at a time (16-byte accesses for fp32, at element alignment: rows start wherever the
// leading dimension puts them).  Row sums are fp32 per thread (a few hundred terms), combined over the block in
// fp32 and over the blocks of a row in fp64, in a fixed order: the same input gives the same bits on every run.
#include "common.hpp"

namespace aprnet {

constexpr int NTB = 256;           // threads per block
constexpr int NORM_BLOCKS = 256;   // blocks per row in the two reductions (upper bound)
constexpr int NORM_EPT = 16;       // elements per thread in the two elementwise kernels

template <typename T> struct Quad { T v[4]; };     // alignment of one element

// Block-wide sum of two values per thread -> thread 0 of the block holds the result.
__device__ __forceinline__ void block_sum2(float& a, float& b) {
    __shared__ float red[2][NTB / 64];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { a += __shfl_down(a, off); b += __shfl_down(b, off); }
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = a; red[1][threadIdx.x >> 6] = b; }
    __syncthreads();
    if (threadIdx.x == 0) {
        a = b = 0.f;
#pragma unroll
        for (int w = 0; w < NTB / 64; ++w) { a += red[0][w]; b += red[1][w]; }
    }
}

// partial[(row * gridDim.x + block) * 2 + {0, 1}] = sum (x - K), sum (x - K)^2 over the block's elements, K = row[0]
template <typename T>
__global__ void __launch_bounds__(NTB)
row_moments_partial_kernel(const T* __restrict__ x, int64_t ldx, int64_t n, float* __restrict__ partial) {
    const T* row = x + (int64_t)blockIdx.y * ldx;
    const float K = Num<T>::ld(row[0]);
    float s1a = 0.f, s2a = 0.f, s1b = 0.f, s2b = 0.f;
    const int64_t nq = n >> 2, stride = (int64_t)gridDim.x * NTB;
    int64_t q = (int64_t)blockIdx.x * NTB + threadIdx.x;
    for (; q + stride < nq; q += 2 * stride) {
        const Quad<T> u = reinterpret_cast<const Quad<T>*>(row)[q], w = reinterpret_cast<const Quad<T>*>(row)[q + stride];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float du = Num<T>::ld(u.v[k]) - K, dw = Num<T>::ld(w.v[k]) - K;
            s1a += du; s2a += du * du; s1b += dw; s2b += dw * dw;
        }
    }
    if (q < nq) {
        const Quad<T> u = reinterpret_cast<const Quad<T>*>(row)[q];
#pragma unroll
        for (int k = 0; k < 4; ++k) { const float du = Num<T>::ld(u.v[k]) - K; s1a += du; s2a += du * du; }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const float du = Num<T>::ld(row[4 * nq + threadIdx.x]) - K; s1b += du; s2b += du * du;
    }
    float s1 = s1a + s1b, s2 = s2a + s2b;
    block_sum2(s1, s2);
    if (threadIdx.x == 0) {
        float* p = partial + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 2;
        p[0] = s1; p[1] = s2;
    }
}

// One wave per row: the partial sums of its blocks in fp64 -> mean, sum of squared deviations.
template <typename T>
__global__ void __launch_bounds__(64)
row_moments_final_kernel(const T* __restrict__ x, int64_t ldx, int64_t n, const float* __restrict__ partial, int nb,
                         double* __restrict__ mean, double* __restrict__ m2) {
    const int64_t r = blockIdx.x;
    double s1 = 0, s2 = 0;
    for (int i = threadIdx.x; i < nb; i += 64) { s1 += partial[(r * nb + i) * 2]; s2 += partial[(r * nb + i) * 2 + 1]; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { s1 += __shfl_down(s1, off); s2 += __shfl_down(s2, off); }
    if (threadIdx.x == 0) {
        const double K = (double)Num<T>::ld(x[r * ldx]);
        mean[r] = K + s1 / (double)n;
        m2[r] = fmax(s2 - s1 * s1 / (double)n, 0.0);
    }
}

template <typename T, bool RELU>
__global__ void __launch_bounds__(NTB)
norm_apply_kernel(const T* __restrict__ x, int64_t ldx, int64_t n, const float* __restrict__ mean,
                  const float* __restrict__ scale, const float* __restrict__ shift, T* __restrict__ y, int64_t ldy) {
    const int r = blockIdx.y;
    const T* xr = x + (int64_t)r * ldx;
    T* yr = y + (int64_t)r * ldy;
    const float m = mean[r], sc = scale[r], sh = shift[r];
    const int64_t nq = n >> 2, q0 = (int64_t)blockIdx.x * (NTB * NORM_EPT / 4) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < NORM_EPT / 4; ++k) {
        const int64_t q = q0 + k * NTB;
        if (q >= nq) break;
        const Quad<T> u = reinterpret_cast<const Quad<T>*>(xr)[q];
        Quad<T> o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float v = (Num<T>::ld(u.v[j]) - m) * sc + sh;
            if (RELU) v = v > 0.f ? v : 0.f;            // NaN -> 0 differs from torch only for NaN inputs
            o.v[j] = Num<T>::st(v);
        }
        reinterpret_cast<Quad<T>*>(yr)[q] = o;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = 4 * nq + threadIdx.x;
        float v = (Num<T>::ld(xr[i]) - m) * sc + sh;
        if (RELU) v = v > 0.f ? v : 0.f;
        yr[i] = Num<T>::st(v);
    }
}

// partial[...] = sum g, sum g * xhat;  g = gy where y > 0 (RELU) or gy,  xhat = (x - mean) * rstd
template <typename T, bool RELU>
__global__ void __launch_bounds__(NTB)
norm_bwd_sums_partial_kernel(const T* __restrict__ gy, int64_t ldg, const T* __restrict__ x, int64_t ldx,
                             const T* __restrict__ y, int64_t ldy, int64_t n, const float* __restrict__ mean,
                             const float* __restrict__ rstd, float* __restrict__ partial) {
    const int r = blockIdx.y;
    const T* gr = gy + (int64_t)r * ldg;
    const T* xr = x + (int64_t)r * ldx;
    const T* yr = RELU ? y + (int64_t)r * ldy : nullptr;
    const float m = mean[r], rs = rstd[r];
    float s1 = 0.f, s2 = 0.f;
    const int64_t nq = n >> 2, stride = (int64_t)gridDim.x * NTB;
    for (int64_t q = (int64_t)blockIdx.x * NTB + threadIdx.x; q < nq; q += stride) {
        const Quad<T> g = reinterpret_cast<const Quad<T>*>(gr)[q], u = reinterpret_cast<const Quad<T>*>(xr)[q];
        Quad<T> o;
        if (RELU) o = reinterpret_cast<const Quad<T>*>(yr)[q];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float gv = Num<T>::ld(g.v[j]);
            if (RELU) gv = Num<T>::ld(o.v[j]) > 0.f ? gv : 0.f;
            s1 += gv; s2 += gv * ((Num<T>::ld(u.v[j]) - m) * rs);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = 4 * nq + threadIdx.x;
        float gv = Num<T>::ld(gr[i]);
        if (RELU) gv = Num<T>::ld(yr[i]) > 0.f ? gv : 0.f;
        s1 += gv; s2 += gv * ((Num<T>::ld(xr[i]) - m) * rs);
    }
    block_sum2(s1, s2);
    if (threadIdx.x == 0) {
        float* p = partial + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * 2;
        p[0] = s1; p[1] = s2;
    }
}

__global__ void __launch_bounds__(64)
norm_sums_final_kernel(const float* __restrict__ partial, int nb, double* __restrict__ out0, double* __restrict__ out1) {
    const int64_t r = blockIdx.x;
    double s1 = 0, s2 = 0;
    for (int i = threadIdx.x; i < nb; i += 64) { s1 += partial[(r * nb + i) * 2]; s2 += partial[(r * nb + i) * 2 + 1]; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) { s1 += __shfl_down(s1, off); s2 += __shfl_down(s2, off); }
    if (threadIdx.x == 0) { out0[r] = s1; out1[r] = s2; }
}

template <typename T, bool RELU>
__global__ void __launch_bounds__(NTB)
norm_bwd_apply_kernel(const T* __restrict__ gy, int64_t ldg, const T* __restrict__ x, int64_t ldx,
                      const T* __restrict__ y, int64_t ldy, int64_t n, const float* __restrict__ mean,
                      const float* __restrict__ rstd, const float* __restrict__ ca, const float* __restrict__ cb,
                      const float* __restrict__ cc, T* __restrict__ gx, int64_t ldo) {
    const int r = blockIdx.y;
    const T* gr = gy + (int64_t)r * ldg;
    const T* xr = x + (int64_t)r * ldx;
    const T* yr = RELU ? y + (int64_t)r * ldy : nullptr;
    T* outr = gx + (int64_t)r * ldo;
    const float m = mean[r], rs = rstd[r], a = ca[r], b = cb[r], c = cc[r];
    const int64_t nq = n >> 2, q0 = (int64_t)blockIdx.x * (NTB * NORM_EPT / 4) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < NORM_EPT / 4; ++k) {
        const int64_t q = q0 + k * NTB;
        if (q >= nq) break;
        const Quad<T> g = reinterpret_cast<const Quad<T>*>(gr)[q], u = reinterpret_cast<const Quad<T>*>(xr)[q];
        Quad<T> o, res;
        if (RELU) o = reinterpret_cast<const Quad<T>*>(yr)[q];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float gv = Num<T>::ld(g.v[j]);
            if (RELU) gv = Num<T>::ld(o.v[j]) > 0.f ? gv : 0.f;
            res.v[j] = Num<T>::st(a * gv + b * ((Num<T>::ld(u.v[j]) - m) * rs) + c);
        }
        reinterpret_cast<Quad<T>*>(outr)[q] = res;
    }
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const int64_t i = 4 * nq + threadIdx.x;
        float gv = Num<T>::ld(gr[i]);
        if (RELU) gv = Num<T>::ld(yr[i]) > 0.f ? gv : 0.f;
        outr[i] = Num<T>::st(a * gv + b * ((Num<T>::ld(xr[i]) - m) * rs) + c);
    }
}

// ---------------------------------------------------------------------------- joining rows into sets
// One thread per row r = b * C + c.  The rows that share statistics with it ("its set") are the rows of channel c
// over the batch (groups == 0: BatchNorm) or the C / groups rows of its group in batch item b (GroupNorm); every
// thread joins its own set (a few to a few hundred values), which keeps the whole join in one tiny launch.
struct SetOf {
    int first, stride, count;       // member j is row first + j * stride
};
__device__ __forceinline__ SetOf set_of(int r, int B, int C, int groups) {
    if (groups == 0) return SetOf{r % C, C, B};
    const int k = C / groups;
    return SetOf{(r / k) * k, 1, k};
}

// Per-row coefficients of the forward pass from the per-row moments (or from given statistics per channel).
__global__ void norm_coeffs_fwd_kernel(int B, int C, int groups, double n, double eps, const double* __restrict__ row_mean,
                                       const double* __restrict__ row_m2, const float* __restrict__ given_mean,
                                       const float* __restrict__ given_var, const float* __restrict__ gamma,
                                       const float* __restrict__ beta, float* __restrict__ mean32, float* __restrict__ rstd32,
                                       float* __restrict__ scale32, float* __restrict__ shift32, float* __restrict__ set_mean,
                                       float* __restrict__ set_var) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= B * C) return;
    const int c = r % C;
    double mean, var;
    if (given_mean) {
        mean = given_mean[c]; var = given_var[c];
    } else {
        const SetOf s = set_of(r, B, C, groups);
        double sm = 0;
        for (int j = 0; j < s.count; ++j) sm += row_mean[s.first + j * s.stride];
        mean = sm / s.count;
        double m2 = 0;
        for (int j = 0; j < s.count; ++j) {
            const double d = row_mean[s.first + j * s.stride] - mean;
            m2 += row_m2[s.first + j * s.stride] + n * d * d;
        }
        var = m2 / (n * s.count);
        if (r == s.first) {             // the set's first row reports the statistics
            const int si = groups == 0 ? c : r / (C / groups);
            set_mean[si] = (float)mean; set_var[si] = (float)var;
        }
    }
    const double rstd = 1.0 / sqrt(var + eps);
    mean32[r] = (float)mean; rstd32[r] = (float)rstd;
    scale32[r] = (float)((gamma ? (double)gamma[c] : 1.0) * rstd);
    shift32[r] = beta ? beta[c] : 0.f;
}

// Per-row coefficients of gx = a * g + b * xhat + c from the per-row sums, and the parameter gradients.
__global__ void norm_coeffs_bwd_kernel(int B, int C, int groups, double n, int own_stats, const double* __restrict__ sum_g,
                                       const double* __restrict__ sum_gx, const float* __restrict__ gamma,
                                       const float* __restrict__ rstd32, float* __restrict__ ca, float* __restrict__ cb,
                                       float* __restrict__ cc, float* __restrict__ grad_gamma, float* __restrict__ grad_beta) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= B * C) return;
    const int c = r % C;
    const double rs = rstd32[r];
    double g1 = 0, g2 = 0;
    if (own_stats) {                    // the statistics depend on the input: set means of gamma * g and gamma * g * xhat
        const SetOf s = set_of(r, B, C, groups);
        for (int j = 0; j < s.count; ++j) {
            const int m = s.first + j * s.stride;
            const double gm = gamma ? (double)gamma[m % C] : 1.0;
            g1 += gm * sum_g[m]; g2 += gm * sum_gx[m];
        }
        g1 /= n * s.count; g2 /= n * s.count;
    }
    ca[r] = (float)((gamma ? (double)gamma[c] : 1.0) * rs);
    cb[r] = (float)(-rs * g2);
    cc[r] = (float)(-rs * g1);
    if (r < C && (grad_gamma || grad_beta)) {       // sums over the batch for channel c = r
        double sg = 0, sgx = 0;
        for (int b = 0; b < B; ++b) { sg += sum_g[b * C + r]; sgx += sum_gx[b * C + r]; }
        if (grad_gamma) grad_gamma[r] = (float)sgx;
        if (grad_beta) grad_beta[r] = (float)sg;
    }
}

// ---------------------------------------------------------------------------- host side
static int check_rows(const char* what, int64_t rows, int64_t n) {
    if (rows < 0 || rows > 65535) return fail(APRNET_ERR_INVALID_ARGUMENT, what);      // rows ride on gridDim.y
    if (n <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, what);
    return 0;
}
static unsigned reduce_blocks(int64_t n) { return (unsigned)std::min<int64_t>(NORM_BLOCKS, std::max<int64_t>(1, n / (4 * NTB * 4))); }
static unsigned stream_blocks(int64_t n) { return (unsigned)((n / 4 + NTB * NORM_EPT / 4 - 1) / (NTB * NORM_EPT / 4)) + (n < 4); }

template <typename T>
int row_moments(const T* x, int64_t ldx, int64_t rows, int64_t n, double* mean, double* m2, float* work, hipStream_t st) {
    if (int rc = check_rows("row_moments: rows must be in [0, 65535] and n positive", rows, n)) return rc;
    if (rows == 0) return 0;
    if (!x || !mean || !m2 || !work || ldx < n) return fail(APRNET_ERR_INVALID_ARGUMENT, "row_moments: null argument or ldx < n");
    const unsigned nb = reduce_blocks(n);
    hipLaunchKernelGGL(row_moments_partial_kernel<T>, dim3(nb, (unsigned)rows), dim3(NTB), 0, st, x, ldx, n, work);
    hipLaunchKernelGGL(row_moments_final_kernel<T>, dim3((unsigned)rows), dim3(64), 0, st, x, ldx, n, work, (int)nb, mean, m2);
    APRNET_LAUNCH_CHECK("row_moments kernels");
    return 0;
}

template <typename T>
int norm_apply(const T* x, int64_t ldx, int64_t rows, int64_t n, const float* mean, const float* scale, const float* shift,
               int relu, T* y, int64_t ldy, hipStream_t st) {
    if (int rc = check_rows("norm_apply: rows must be in [0, 65535] and n positive", rows, n)) return rc;
    if (rows == 0) return 0;
    if (!x || !y || !mean || !scale || !shift || ldx < n || ldy < n)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "norm_apply: null argument or leading dimension < n");
    const dim3 grid(stream_blocks(n), (unsigned)rows);
    if (relu) hipLaunchKernelGGL((norm_apply_kernel<T, true>), grid, dim3(NTB), 0, st, x, ldx, n, mean, scale, shift, y, ldy);
    else hipLaunchKernelGGL((norm_apply_kernel<T, false>), grid, dim3(NTB), 0, st, x, ldx, n, mean, scale, shift, y, ldy);
    APRNET_LAUNCH_CHECK("norm_apply_kernel");
    return 0;
}

template <typename T>
int norm_bwd_sums(const T* gy, int64_t ldg, const T* x, int64_t ldx, const T* y, int64_t ldy, int64_t rows, int64_t n,
                  const float* mean, const float* rstd, double* sum_g, double* sum_gx, float* work, hipStream_t st) {
    if (int rc = check_rows("norm_bwd_sums: rows must be in [0, 65535] and n positive", rows, n)) return rc;
    if (rows == 0) return 0;
    if (!gy || !x || !mean || !rstd || !sum_g || !sum_gx || !work || ldg < n || ldx < n || (y && ldy < n))
        return fail(APRNET_ERR_INVALID_ARGUMENT, "norm_bwd_sums: null argument or leading dimension < n");
    const unsigned nb = reduce_blocks(n);
    const dim3 grid(nb, (unsigned)rows);
    if (y) hipLaunchKernelGGL((norm_bwd_sums_partial_kernel<T, true>), grid, dim3(NTB), 0, st, gy, ldg, x, ldx, y, ldy, n, mean, rstd, work);
    else hipLaunchKernelGGL((norm_bwd_sums_partial_kernel<T, false>), grid, dim3(NTB), 0, st, gy, ldg, x, ldx, y, ldy, n, mean, rstd, work);
    hipLaunchKernelGGL(norm_sums_final_kernel, dim3((unsigned)rows), dim3(64), 0, st, work, (int)nb, sum_g, sum_gx);
    APRNET_LAUNCH_CHECK("norm_bwd_sums kernels");
    return 0;
}

template <typename T>
int norm_bwd_apply(const T* gy, int64_t ldg, const T* x, int64_t ldx, const T* y, int64_t ldy, int64_t rows, int64_t n,
                   const float* mean, const float* rstd, const float* a, const float* b, const float* c, T* gx, int64_t ldo,
                   hipStream_t st) {
    if (int rc = check_rows("norm_bwd_apply: rows must be in [0, 65535] and n positive", rows, n)) return rc;
    if (rows == 0) return 0;
    if (!gy || !x || !mean || !rstd || !a || !b || !c || !gx || ldg < n || ldx < n || ldo < n || (y && ldy < n))
        return fail(APRNET_ERR_INVALID_ARGUMENT, "norm_bwd_apply: null argument or leading dimension < n");
    const dim3 grid(stream_blocks(n), (unsigned)rows);
    if (y) hipLaunchKernelGGL((norm_bwd_apply_kernel<T, true>), grid, dim3(NTB), 0, st, gy, ldg, x, ldx, y, ldy, n, mean, rstd, a, b, c, gx, ldo);
    else hipLaunchKernelGGL((norm_bwd_apply_kernel<T, false>), grid, dim3(NTB), 0, st, gy, ldg, x, ldx, y, ldy, n, mean, rstd, a, b, c, gx, ldo);
    APRNET_LAUNCH_CHECK("norm_bwd_apply_kernel");
    return 0;
}

static int check_sets(const char* what, int B, int C, int groups, int64_t n) {
    if (B <= 0 || C <= 0 || n <= 0 || (int64_t)B * C > 65535 || groups < 0 || (groups > 0 && C % groups != 0))
        return fail(APRNET_ERR_INVALID_ARGUMENT, what);
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
int aprnet_norm_coeffs_fwd(int B, int C, int groups, int64_t n, double eps, const double* row_mean, const double* row_m2,
                           const float* given_mean, const float* given_var, const float* gamma, const float* beta,
                           float* mean32, float* rstd32, float* scale32, float* shift32, float* set_mean, float* set_var,
                           void* st) {
    if (int rc = check_sets("norm_coeffs_fwd: B, C, n positive, B * C <= 65535, groups dividing C", B, C, groups, n)) return rc;
    const bool given = given_mean && given_var;
    if (!mean32 || !rstd32 || !scale32 || !shift32 || (!given && (!row_mean || !row_m2 || !set_mean || !set_var)))
        return fail(APRNET_ERR_INVALID_ARGUMENT, "norm_coeffs_fwd: null argument");
    hipLaunchKernelGGL(norm_coeffs_fwd_kernel, dim3((unsigned)((B * C + 127) / 128)), dim3(128), 0, (hipStream_t)st, B, C, groups,
                       (double)n, eps, row_mean, row_m2, given ? given_mean : nullptr, given ? given_var : nullptr, gamma, beta,
                       mean32, rstd32, scale32, shift32, set_mean, set_var);
    APRNET_LAUNCH_CHECK("norm_coeffs_fwd_kernel");
    return 0;
}
int aprnet_norm_coeffs_bwd(int B, int C, int groups, int64_t n, int own_stats, const double* sum_g, const double* sum_gx,
                           const float* gamma, const float* rstd32, float* a, float* b, float* c, float* grad_gamma,
                           float* grad_beta, void* st) {
    if (int rc = check_sets("norm_coeffs_bwd: B, C, n positive, B * C <= 65535, groups dividing C", B, C, groups, n)) return rc;
    if (!sum_g || !sum_gx || !rstd32 || !a || !b || !c) return fail(APRNET_ERR_INVALID_ARGUMENT, "norm_coeffs_bwd: null argument");
    hipLaunchKernelGGL(norm_coeffs_bwd_kernel, dim3((unsigned)((B * C + 127) / 128)), dim3(128), 0, (hipStream_t)st, B, C, groups,
                       (double)n, own_stats, sum_g, sum_gx, gamma, rstd32, a, b, c, grad_gamma, grad_beta);
    APRNET_LAUNCH_CHECK("norm_coeffs_bwd_kernel");
    return 0;
}
int64_t aprnet_norm_work_elems(int64_t rows) { return std::max<int64_t>(rows, 1) * NORM_BLOCKS * 2; }
#define NORM_API(T, CT, SFX)                                                                                            \
    int aprnet_row_moments_##SFX(const CT* x, int64_t ldx, int64_t rows, int64_t n, double* mean, double* m2, float* work, \
                                 void* st) {                                                                            \
        return row_moments<T>((const T*)x, ldx, rows, n, mean, m2, work, (hipStream_t)st); }                            \
    int aprnet_norm_apply_##SFX(const CT* x, int64_t ldx, int64_t rows, int64_t n, const float* mean, const float* scale, \
                                const float* shift, int relu, CT* y, int64_t ldy, void* st) {                           \
        return norm_apply<T>((const T*)x, ldx, rows, n, mean, scale, shift, relu, (T*)y, ldy, (hipStream_t)st); }       \
    int aprnet_norm_bwd_sums_##SFX(const CT* gy, int64_t ldg, const CT* x, int64_t ldx, const CT* y, int64_t ldy,       \
                                   int64_t rows, int64_t n, const float* mean, const float* rstd, double* sum_g,        \
                                   double* sum_gx, float* work, void* st) {                                             \
        return norm_bwd_sums<T>((const T*)gy, ldg, (const T*)x, ldx, (const T*)y, ldy, rows, n, mean, rstd, sum_g,      \
                                sum_gx, work, (hipStream_t)st); }                                                       \
    int aprnet_norm_bwd_apply_##SFX(const CT* gy, int64_t ldg, const CT* x, int64_t ldx, const CT* y, int64_t ldy,      \
                                    int64_t rows, int64_t n, const float* mean, const float* rstd, const float* a,      \
                                    const float* b, const float* c, CT* gx, int64_t ldo, void* st) {                    \
        return norm_bwd_apply<T>((const T*)gy, ldg, (const T*)x, ldx, (const T*)y, ldy, rows, n, mean, rstd, a, b, c,   \
                                 (T*)gx, ldo, (hipStream_t)st); }
NORM_API(float, float, f32)
NORM_API(bf16_t, uint16_t, bf16)
}
