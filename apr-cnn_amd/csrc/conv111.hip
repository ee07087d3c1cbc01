// 1x1x1 convolution: Convolution<1,1,1>::forward/backward (conv.hpp:199-256, 484-554).
// Particles of one level are contiguous in the feature vector (conv111_gpu.cu:30-31), and so are the
// downsampled particles, so the operator is a per-segment channel GEMM: out[co][i] = sum_ci w[s][co][ci] x[ci][i]
// with the stencil index s = min(S-1, Lc-level) constant per segment.  One launch per segment keeps
// the weights wave-uniform (scalar loads); x is read once per block of COB output channels.
#include "common.hpp"

namespace aprnet {

constexpr int TB1 = 256;

// dst[o][i] = sum_c W(o, c) * src[c][i],  W(o, c) = w[o * so + c * sc]
// T = storage type of the features; weights, bias and sums in Num<T>::acc (fp32 for bfloat16 features)
template <typename T, int OB>
__global__ void __launch_bounds__(TB1)
conv111_kernel(const T* __restrict__ src, int64_t lds, int Csrc, const typename Num<T>::acc* __restrict__ w, int so, int sc,
               const typename Num<T>::acc* __restrict__ bias, T* __restrict__ dst, int64_t ldd, int Cdst, int64_t begin, int64_t end,
               int relu) {
    typedef typename Num<T>::acc A;
    const int64_t i = begin + (int64_t)blockIdx.x * TB1 + threadIdx.x;
    if (i >= end) return;
    const int o0 = blockIdx.y * OB;
    A acc[OB];
#pragma unroll
    for (int o = 0; o < OB; ++o) acc[o] = 0;
    constexpr int CU = 8;            // input channels loaded together: eight independent loads in flight
    for (int c0 = 0; c0 < Csrc; c0 += CU) {
        A v[CU];
#pragma unroll
        for (int k = 0; k < CU; ++k) v[k] = c0 + k < Csrc ? Num<T>::ld(src[(int64_t)(c0 + k) * lds + i]) : (A)0;
#pragma unroll
        for (int k = 0; k < CU; ++k) {
            if (c0 + k >= Csrc) break;
#pragma unroll
            for (int o = 0; o < OB; ++o)
                if (o0 + o < Cdst) acc[o] += w[(int64_t)(o0 + o) * so + (int64_t)(c0 + k) * sc] * v[k];
        }
    }
#pragma unroll
    for (int o = 0; o < OB; ++o)
        if (o0 + o < Cdst) {
            A v = acc[o] + (bias ? bias[o0 + o] : (A)0);
            if (relu) v = v < (A)0 ? (A)0 : v;
            dst[(int64_t)(o0 + o) * ldd + i] = Num<T>::st(v);
        }
}

// The same product on the matrix cores (fp32): M = 32 outputs, N = 32 positions, K = input channels two at a
// time.  v_mfma_f32_32x32x2_f32 takes  A: lane l -> W(o = l%32, c = 2p + l/32)  (kept in registers for the
// whole kernel) and  B: lane l -> src[c = 2p + l/32][i0 + l%32]  (two coalesced 128-byte rows per load), so
// the kernel streams the input once per 32 output channels and is bound by HBM.
typedef float floatx16_111 __attribute__((ext_vector_type(16)));
template <typename T> struct Pair111 { T v[2]; };        // two neighbours, alignment of one element
template <int BYTES> struct PairBits111;
template <> struct PairBits111<4> { typedef uint32_t type __attribute__((aligned(2))); };
template <> struct PairBits111<8> { typedef uint32_t type __attribute__((ext_vector_type(2), aligned(4))); };

// T = storage type of the features (float, or bfloat16 with fp32 weights, bias and arithmetic)
template <typename T, int KP>      // KP = channel pairs held in registers (ceil(Csrc / 2) <= KP)
__global__ void __launch_bounds__(TB1) __attribute__((amdgpu_waves_per_eu(KP <= 16 ? 2 : 1)))
conv111_mfma_kernel(const T* __restrict__ src, int64_t lds, int Csrc, const float* __restrict__ w, int so, int sc,
                    const float* __restrict__ bias, T* __restrict__ dst, int64_t ldd, int Cdst, int64_t begin,
                    int64_t end, int relu) {
    const int lane = threadIdx.x & 63, hi = lane >> 5, col = lane & 31;
    const int o0 = blockIdx.y * 32;
    // weights and bias: all loads first, from clamped places, masked afterwards (a load under a per-lane branch is
    // waited for on the spot: 32 round trips in a row at the start of every block)
    float aw[KP];
    {
        const int o = min(o0 + col, Cdst - 1);
#pragma unroll
        for (int p = 0; p < KP; ++p) aw[p] = w[(int64_t)o * so + (int64_t)min(2 * p + hi, Csrc - 1) * sc];
#pragma unroll
        for (int p = 0; p < KP; ++p) aw[p] = (2 * p + hi < Csrc && o0 + col < Cdst) ? aw[p] : 0.f;
    }
    float bs[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) bs[r] = bias ? bias[min(o0 + 8 * (r >> 2) + 4 * hi + (r & 3), Cdst - 1)] : 0.f;
    const int64_t nwave = (int64_t)gridDim.x * (TB1 / 64);
    const int64_t wave = (int64_t)blockIdx.x * (TB1 / 64) + (threadIdx.x >> 6);
    for (int64_t i0 = begin + wave * 64; i0 < end; i0 += nwave * 64) {
        if (i0 + 64 <= end) {
            // whole block of 64 positions: lane `col` takes the neighbours i0 + 2 col and i0 + 2 col + 1 as one
            // (element-aligned) pair, so a half-wave reads and writes 32 pairs in a row per channel
            typedef typename PairBits111<2 * sizeof(T)>::type B;
            const int64_t ip = i0 + 2 * col;
            // Every channel pair is loaded, none under a branch: the channel depends on the lane's half, and before a
            // load under a per-lane branch the compiler waits for all loads in flight, which made the channels of a
            // block sixteen memory round trips in a row.  A pair past the last channel re-reads the last one; its
            // weights are zero.  (One vector value each way: a struct of two elements is split into two accesses.)
            B raw[KP];
#pragma unroll
            for (int p = 0; p < KP; ++p) {
                const int c = min(2 * p + hi, Csrc - 1);
                raw[p] = *reinterpret_cast<const B*>(src + (int64_t)c * lds + ip);
            }
            if constexpr (KP <= 32) __builtin_amdgcn_sched_barrier(0);      // all loads in flight before the first matrix instruction
            float va[KP], vb[KP];
#pragma unroll
            for (int p = 0; p < KP; ++p) {
                const Pair111<T> pv = __builtin_bit_cast(Pair111<T>, raw[p]);
                va[p] = Num<T>::ld(pv.v[0]); vb[p] = Num<T>::ld(pv.v[1]);
            }
            floatx16_111 acca, accb;
#pragma unroll
            for (int r = 0; r < 16; ++r) { acca[r] = bs[r]; accb[r] = bs[r]; }
#pragma unroll
            for (int p = 0; p < KP; ++p) {
                acca = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[p], va[p], acca, 0, 0, 0);
                accb = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[p], vb[p], accb, 0, 0, 0);
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int o = o0 + 8 * (r >> 2) + 4 * hi + (r & 3);
                if (o < Cdst) {
                    float ya = acca[r], yb = accb[r];
                    if (relu) { ya = ya < 0.f ? 0.f : ya; yb = yb < 0.f ? 0.f : yb; }
                    Pair111<T> pv;
                    pv.v[0] = Num<T>::st(ya); pv.v[1] = Num<T>::st(yb);
                    *reinterpret_cast<B*>(dst + (int64_t)o * ldd + ip) = __builtin_bit_cast(B, pv);
                }
            }
            continue;
        }
        const int64_t ia = i0 + col, ib = i0 + 32 + col;
        float va[KP], vb[KP];
#pragma unroll
        for (int p = 0; p < KP; ++p) {
            const int c = 2 * p + hi;
            const T* row = src + (int64_t)c * lds;
            va[p] = (c < Csrc && ia < end) ? Num<T>::ld(row[ia]) : 0.f;
            vb[p] = (c < Csrc && ib < end) ? Num<T>::ld(row[ib]) : 0.f;
        }
        floatx16_111 acca, accb;
#pragma unroll
        for (int r = 0; r < 16; ++r) { acca[r] = bs[r]; accb[r] = bs[r]; }
#pragma unroll
        for (int p = 0; p < KP; ++p) {
            acca = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[p], va[p], acca, 0, 0, 0);
            accb = __builtin_amdgcn_mfma_f32_32x32x2f32(aw[p], vb[p], accb, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int o = o0 + 8 * (r >> 2) + 4 * hi + (r & 3);
            if (o < Cdst) {
                float ya = acca[r], yb = accb[r];
                if (relu) { ya = ya < 0.f ? 0.f : ya; yb = yb < 0.f ? 0.f : yb; }
                if (ia < end) dst[(int64_t)o * ldd + ia] = Num<T>::st(ya);
                if (ib < end) dst[(int64_t)o * ldd + ib] = Num<T>::st(yb);
            }
        }
    }
}

// dispatch on the number of channel pairs kept in registers; false when the layer is too wide for this kernel
template <typename T>
static bool launch_conv111_mfma(const T* src, int64_t lds, int Csrc, const float* w, int so, int sc, const float* bias,
                                T* dst, int64_t ldd, int Cdst, int64_t begin, int64_t end, hipStream_t st, int relu = 0) {
    const int kp = (Csrc + 1) / 2;
    const int64_t n = end - begin;
    dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 256 * 8), (unsigned)((Cdst + 31) / 32));
#define APRNET_111(KP) hipLaunchKernelGGL((conv111_mfma_kernel<T, KP>), grid, dim3(TB1), 0, st, src, lds, Csrc, w, so, sc, bias, \
                                          dst, ldd, Cdst, begin, end, relu)
    if (kp <= 8) APRNET_111(8);
    else if (kp <= 16) APRNET_111(16);
    else if (kp <= 32) APRNET_111(32);
    else if (kp <= 64) APRNET_111(64);
    else return false;
#undef APRNET_111
    return true;
}
template <typename T>
static bool try_conv111_mfma(const T*, int64_t, int, const T*, int, int, const T*, T*, int64_t, int, int64_t, int64_t, hipStream_t,
                             int = 0) {
    return false;
}
int conv_path();
template <>
bool try_conv111_mfma<float>(const float* src, int64_t lds, int Csrc, const float* w, int so, int sc, const float* bias,
                             float* dst, int64_t ldd, int Cdst, int64_t begin, int64_t end, hipStream_t st, int relu) {
    if (conv_path() == 1) return false;
    return launch_conv111_mfma<float>(src, lds, Csrc, w, so, sc, bias, dst, ldd, Cdst, begin, end, st, relu);
}

// gw[co][ci] += sum_i gy[co][i] * x[ci][i] over [begin, end): 8x8 register tile per thread, block
// reduction through LDS; then one atomic per (co, ci) and block, or - with `part` - the block's sum goes to
// part[blockIdx.x][co][ci] for conv111_dw_reduce_kernel to add up in a fixed order (same bits on every run).
template <typename T>
__global__ void __launch_bounds__(TB1)
conv111_dw_kernel(const T* __restrict__ x, int64_t ldx, int Cin, const T* __restrict__ gy, int64_t ldy, int Cout,
                  typename Num<T>::acc* __restrict__ gw, typename Num<T>::acc* __restrict__ part, int64_t begin, int64_t end) {
    typedef typename Num<T>::acc A;          // bfloat16 features: fp32 products, sums and weight gradient
    constexpr int B = 8;
    __shared__ A red[TB1 / 64][B * B];
    const int co0 = blockIdx.y * B, ci0 = blockIdx.z * B;
    A acc[B][B];
#pragma unroll
    for (int a = 0; a < B; ++a)
#pragma unroll
        for (int b = 0; b < B; ++b) acc[a][b] = 0;
    for (int64_t i = begin + (int64_t)blockIdx.x * TB1 + threadIdx.x; i < end; i += (int64_t)gridDim.x * TB1) {
        A g[B], v[B];
#pragma unroll
        for (int a = 0; a < B; ++a) g[a] = co0 + a < Cout ? Num<T>::ld(gy[(int64_t)(co0 + a) * ldy + i]) : (A)0;
#pragma unroll
        for (int b = 0; b < B; ++b) v[b] = ci0 + b < Cin ? Num<T>::ld(x[(int64_t)(ci0 + b) * ldx + i]) : (A)0;
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
            A s = acc[a][b];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) s += __shfl_down(s, off);
            if (lane == 0) red[wave][a * B + b] = s;
        }
    __syncthreads();
    if (threadIdx.x < B * B) {
        A s = 0;
#pragma unroll
        for (int wv = 0; wv < TB1 / 64; ++wv) s += red[wv][threadIdx.x];
        const int a = threadIdx.x / B, b = threadIdx.x % B;
        if (co0 + a < Cout && ci0 + b < Cin) {
            const int64_t e = (int64_t)(co0 + a) * Cin + (ci0 + b);
            if (part) part[(int64_t)blockIdx.x * Cout * Cin + e] = s;
            else atomicAdd(&gw[e], s);
        }
    }
}

// gw[e] += part[0][e] + part[1][e] + ... in that order
template <typename A>
__global__ void __launch_bounds__(TB1)
conv111_dw_reduce_kernel(const A* __restrict__ part, int nblocks, int n, A* __restrict__ gw) {
    const int e = blockIdx.x * TB1 + threadIdx.x;
    if (e >= n) return;
    A s = 0;
    for (int b = 0; b < nblocks; ++b) s += part[(int64_t)b * n + e];
    gw[e] += s;
}

int bwd_deterministic();

// the weight gradient of one segment, by partial sums per workgroup (default) or by atomic additions
template <typename T>
static int launch_conv111_dw(aprnet_plan* p, const T* x, int64_t ldx, int Cin, const T* gy, int64_t ldy, int Cout,
                             typename Num<T>::acc* gw, int64_t begin, int64_t end, hipStream_t st) {
    typedef typename Num<T>::acc A;
    const int64_t n = end - begin;
    dim3 g2((unsigned)std::min<int64_t>((n + TB1 * 8 - 1) / (TB1 * 8), 256), (unsigned)((Cout + 7) / 8), (unsigned)((Cin + 7) / 8));
    if (!bwd_deterministic()) {
        hipLaunchKernelGGL(conv111_dw_kernel<T>, g2, dim3(TB1), 0, st, x, ldx, Cin, gy, ldy, Cout, gw, (A*)nullptr, begin, end);
        return 0;
    }
    ScratchLease lease;
    if (int rc = lease.acquire(p, (size_t)g2.x * Cout * Cin * sizeof(A), st)) return rc;
    A* part = (A*)p->d_scratch;
    hipLaunchKernelGGL(conv111_dw_kernel<T>, g2, dim3(TB1), 0, st, x, ldx, Cin, gy, ldy, Cout, gw, part, begin, end);
    hipLaunchKernelGGL(conv111_dw_reduce_kernel<A>, dim3((unsigned)((Cout * Cin + TB1 - 1) / TB1)), dim3(TB1), 0, st, part, (int)g2.x,
                       Cout * Cin, gw);
    return 0;
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
                const T* bias, T* y, int64_t ldy, hipStream_t st, int relu) {
    if (int rc = check_level_delta(p, d, "conv111_forward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv111_forward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv111_forward", "output")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_forward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    // 32 outputs per thread when the layer has more than 16: the input is then read once per 32 output channels
    for (const Segment& sg : segments(p, d, S)) {
        const T* ws = w + (int64_t)sg.stencil * Cout * Cin;
        if (try_conv111_mfma<T>(x, ldx, Cin, ws, Cin, 1, bias, y, ldy, Cout, sg.begin, sg.end, st, relu)) continue;
        if (Cout > 16) {
            dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cout + 31) / 32));
            hipLaunchKernelGGL((conv111_kernel<T, 32>), grid, dim3(TB1), 0, st, x, ldx, Cin, ws, Cin, 1, bias, y, ldy, Cout,
                               sg.begin, sg.end, relu);
        } else {
            dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), 1u);
            hipLaunchKernelGGL((conv111_kernel<T, 16>), grid, dim3(TB1), 0, st, x, ldx, Cin, ws, Cin, 1, bias, y, ldy, Cout,
                               sg.begin, sg.end, relu);
        }
    }
    APRNET_LAUNCH_CHECK("conv111_kernel");
    return 0;
}

template <typename T>
int conv111_bwd(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout, const T* gy,
                int64_t ldy, T* gx, int64_t ldgx, T* gw, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "conv111_backward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv111_backward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv111_backward", "output gradient")) return rc;
    if (int rc = check_rows(ldgx, p->number_parts(d), "conv111_backward", "input gradient")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_backward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    constexpr int OB = 16;
    for (const Segment& sg : segments(p, d, S)) {
        const T* ws = w + (int64_t)sg.stencil * Cout * Cin;
        dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cin + OB - 1) / OB));
        // grad_x[ci][i] = sum_co w[co][ci] * gy[co][i]: the same kernel with the weight strides swapped
        if (!try_conv111_mfma<T>(gy, ldy, Cout, ws, 1, Cin, (const T*)nullptr, gx, ldgx, Cin, sg.begin, sg.end, st))
            hipLaunchKernelGGL((conv111_kernel<T, OB>), grid, dim3(TB1), 0, st, gy, ldy, Cout, ws, 1, Cin, (const T*)nullptr, gx, ldgx, Cin,
                               sg.begin, sg.end, 0);
        if (int rc = launch_conv111_dw<T>(const_cast<aprnet_plan*>(p), x, ldx, Cin, gy, ldy, Cout, gw + (int64_t)sg.stencil * Cout * Cin,
                                          sg.begin, sg.end, st)) return rc;
    }
    APRNET_LAUNCH_CHECK("conv111 backward kernels");
    return 0;
}

int conv111_fwd_bf16(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                     const float* bias, bf16_t* y, int64_t ldy, hipStream_t st, int relu) {
    if (int rc = check_level_delta(p, d, "conv111_forward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv111_forward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv111_forward", "output")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_forward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    for (const Segment& sg : segments(p, d, S))
        if (!launch_conv111_mfma<bf16_t>(x, ldx, Cin, w + (int64_t)sg.stencil * Cout * Cin, Cin, 1, bias, y, ldy, Cout, sg.begin, sg.end, st, relu)) {
            // more than 128 input channels: the vector-ALU kernel (fp32 sums), 16 outputs per thread
            dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cout + 15) / 16));
            hipLaunchKernelGGL((conv111_kernel<bf16_t, 16>), grid, dim3(TB1), 0, st, x, ldx, Cin, w + (int64_t)sg.stencil * Cout * Cin, Cin, 1,
                               bias, y, ldy, Cout, sg.begin, sg.end, relu);
        }
    APRNET_LAUNCH_CHECK("conv111_mfma_kernel");
    return 0;
}

// bfloat16 features and output gradient, fp32 weights and weight gradient (accumulated into gw), fp32 accumulation
int conv111_bwd_bf16(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                     const bf16_t* gy, int64_t ldy, bf16_t* gx, int64_t ldgx, float* gw, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "conv111_backward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv111_backward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv111_backward", "output gradient")) return rc;
    if (int rc = check_rows(ldgx, p->number_parts(d), "conv111_backward", "input gradient")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_backward: empty channel / stencil count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    for (const Segment& sg : segments(p, d, S)) {
        const float* ws = w + (int64_t)sg.stencil * Cout * Cin;
        // grad_x[ci][i] = sum_co w[co][ci] * gy[co][i]: the forward kernel with the weight strides swapped
        if (!launch_conv111_mfma<bf16_t>(gy, ldy, Cout, ws, 1, Cin, nullptr, gx, ldgx, Cin, sg.begin, sg.end, st)) {
            dim3 grid((unsigned)((sg.end - sg.begin + TB1 - 1) / TB1), (unsigned)((Cin + 15) / 16));
            hipLaunchKernelGGL((conv111_kernel<bf16_t, 16>), grid, dim3(TB1), 0, st, gy, ldy, Cout, ws, 1, Cin, (const float*)nullptr, gx, ldgx, Cin,
                               sg.begin, sg.end, 0);
        }
        if (int rc = launch_conv111_dw<bf16_t>(const_cast<aprnet_plan*>(p), x, ldx, Cin, gy, ldy, Cout, gw + (int64_t)sg.stencil * Cout * Cin,
                                               sg.begin, sg.end, st)) return rc;
    }
    APRNET_LAUNCH_CHECK("conv111 backward kernels");
    return 0;
}

// 1x1x1 forward with the optional clamp at zero, for the fused entry points
int conv111_fwd_relu(const aprnet_plan* p, int d, const float* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                     const float* bias, float* y, int64_t ldy, hipStream_t st, int relu) {
    return conv111_fwd<float>(p, d, x, ldx, Cin, w, S, Cout, bias, y, ldy, st, relu);
}
int conv111_fwd_relu(const aprnet_plan* p, int d, const double* x, int64_t ldx, int Cin, const double* w, int S, int Cout,
                     const double* bias, double* y, int64_t ldy, hipStream_t st, int relu) {
    return conv111_fwd<double>(p, d, x, ldx, Cin, w, S, Cout, bias, y, ldy, st, relu);
}
int conv111_fwd_relu(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                     const float* bias, bf16_t* y, int64_t ldy, hipStream_t st, int relu) {
    return conv111_fwd_bf16(p, d, x, ldx, Cin, w, S, Cout, bias, y, ldy, st, relu);
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
int aprnet_conv111_bwd_bf16(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                            const uint16_t* gy, int64_t ldy, uint16_t* gx, int64_t ldgx, float* gw, void* st) {
    return conv111_bwd_bf16(p, d, (const bf16_t*)x, ldx, Cin, w, S, Cout, (const bf16_t*)gy, ldy, (bf16_t*)gx, ldgx, gw, (hipStream_t)st);
}
int aprnet_conv111_fwd_bf16(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int Cin, const float* w, int S,
                            int Cout, const float* bias, uint16_t* y, int64_t ldy, void* st) {
    return conv111_fwd_bf16(p, d, (const bf16_t*)x, ldx, Cin, w, S, Cout, bias, (bf16_t*)y, ldy, (hipStream_t)st, 0);
}
#define CONV111_API(T, SFX)                                                                                        \
    int aprnet_conv111_fwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S,  \
                                 int Cout, const T* bias, T* y, int64_t ldy, void* st) {                            \
        return conv111_fwd<T>(p, d, x, ldx, Cin, w, S, Cout, bias, y, ldy, (hipStream_t)st, 0); }                      \
    int aprnet_conv111_bwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int Cin, const T* w, int S,  \
                                 int Cout, const T* gy, int64_t ldy, T* gx, int64_t ldgx, T* gw, void* st) {        \
        return conv111_bwd<T>(p, d, x, ldx, Cin, w, S, Cout, gy, ldy, gx, ldgx, gw, (hipStream_t)st); }
CONV111_API(float, f32)
CONV111_API(double, f64)
}
