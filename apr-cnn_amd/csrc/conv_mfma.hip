// Stencil convolution forward on the matrix cores (fp32 MFMA), gfx950.
//
// Same tiles, windows and three-source LDS gather as the VALU path (conv_common.hpp); only the
// contraction differs.  For one window the block holds nc output positions ("columns").  The
// contraction  out[co][col] = sum_{ci,t} W[co][ci][t] * patch[ci][pos(col) + off(t)]  is an implicit
// GEMM with M = 32 output channels, N = columns, K = (tap, input channel):
//
//     v_mfma_f32_32x32x2_f32:  D[32x32] += A[32x2] * B[2x32]
//       A: lane l supplies W[co = l%32][k = l/32]        B: lane l supplies patch value of column l%32, k = l/32
//       the two k of one instruction are the two input channels of a pair (ci = 2p, 2p+1), same tap
//
// so every lane owns one column and one channel parity: its B operand for step (p, t) sits at a fixed
// per-lane LDS address plus a compile-time offset (channel-pair stride + tap offset), and its A operand
// likewise in a transposed, padded weight chunk Wl[(c*K + t)][co] that is staged per channel chunk.
// The K loop is fully unrolled: two ds_read_b32 with immediate offsets and one MFMA per step and column
// block, no address arithmetic.  Columns are cut into blocks of 32; wave w owns blocks b with
// (b + rotation) % 4 == w, up to NBW of them, and keeps their 32x32 accumulators in registers across all
// channel chunks, so each output element is written once (no atomics, deterministic).
#include "conv_common.hpp"

namespace aprnet {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Weights are re-laid out once per call into the image the kernel keeps in LDS, so that staging a chunk
// is a straight 16-byte copy:  packed[s][cb][q][(c*K + t)][co]  with co-blocks cb of 32 output channels and
// chunks q of CIB input channels, zero where co or ci run past the layer.
//
// With `transposed` the roles of the two channel axes are swapped and the taps reversed: the image is that
// of the stencil of the input gradient, M = input channels, contraction over (flipped tap, output channel).
// Cm / Ck are the channel counts of the M axis and of the contracted axis.
__global__ void pack_weights_kernel(const float* __restrict__ w, int S_exp, int Cm, int Ck, int K, int CIB,
                                    int transposed, float* __restrict__ out) {
    const int Cout = transposed ? Ck : Cm, Cin = transposed ? Cm : Ck;
    const int ncb = (Cm + 31) / 32, nq = (Ck + CIB - 1) / CIB, KC = CIB * K;
    const int64_t n = (int64_t)S_exp * ncb * nq * KC * 32;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        const int co = (int)(e % 32);
        const int row = (int)((e / 32) % KC);
        const int q = (int)((e / (32 * (int64_t)KC)) % nq);
        const int cb = (int)((e / (32 * (int64_t)KC * nq)) % ncb);
        const int s = (int)(e / (32 * (int64_t)KC * nq * ncb));
        const int c = row / K, t = row - c * K;
        const int ck = q * CIB + c, cm = cb * 32 + co;
        float v = 0.f;
        if (ck < Ck && cm < Cm)
            v = transposed ? w[(((int64_t)s * Cout + ck) * Cin + cm) * K + (K - 1 - t)]
                           : w[(((int64_t)s * Cout + cm) * Cin + ck) * K + t];
        out[e] = v;
    }
}

template <class G>
__device__ __forceinline__ constexpr int tap_offset(int t) {
    return ((t / (G::KX * G::KY)) * G::RX + (t / G::KY) % G::KX) * G::RS + (t % G::KY);
}

// One window for a wave that owns NB of the window's column blocks (blocks b with b % NWAVE == first).
// Every instantiation runs the same staging and the same two barriers per channel chunk, so the waves
// of a block may take different NB (0 included: the wave only helps with the staging).
// MODE 0: forward, results stored (plus bias).  MODE 1: input gradient, results added atomically to the
// place each column names (feature gradient, or tree gradient with COL_TREE).
template <class G, int CIB, int NB, int MODE>
__device__ __forceinline__ void mfma_window(const ConvArgs<float>& a, int co0, int nc, int nitem, bool tree_items, int first,
                                            const float4* __restrict__ wl, const ConvShared<G>& sh,
                                            float* __restrict__ patch, float* __restrict__ Wl,
                                            const float* __restrict__ bias_l) {
    constexpr int WLD = 32;                    // row of the weight chunk: 32 output channels
    constexpr int KC = CIB * G::K;             // k rows per chunk
    const int lane = lane_id();
    constexpr int NBA = NB > 0 ? NB : 1;
    int bbase[NBA];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 5) + (lane & 31);
        const int pos = col < nc ? (int)(sh.col_pos[col] & COL_CELL) - G::TAP0 : 0;
        bbase[j] = pos + (lane >> 5) * G::CH_STRIDE;
    }
    floatx16 acc[NBA];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    const float* ap = Wl + (lane >> 5) * G::K * WLD + (lane & 31);

    // Software pipeline over the channel chunks: the global loads of chunk c+1 (items and weights) are
    // issued into registers before the MFMAs of chunk c and land in LDS after them.
    constexpr int W4 = KC * 8;                                   // float4 elements of a weight chunk
    constexpr int WPT = (W4 + G::NT - 1) / G::NT;
    ItemRegs<G, float, CIB> R;
    float4 wr[WPT];
#define APRNET_LOAD_WEIGHTS(q)                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        wr[k] = (i < W4) ? (wl + (int64_t)(q) * W4)[i] : make_float4(0.f, 0.f, 0.f, 0.f);          \
    }
#define APRNET_STORE_WEIGHTS()                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        if (i < W4) reinterpret_cast<float4*>(Wl)[i] = wr[k];                                      \
    }
    load_items<G, float, CIB>(a, 0, nitem, tree_items, sh, R);
    APRNET_LOAD_WEIGHTS(0)
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    for (int ci0 = 0; ci0 < a.Cin; ci0 += CIB) {
        __syncthreads();            // zeros are in place / the previous chunk's MFMAs have read patch and Wl
        store_items<G, float, CIB>(R, nitem, patch);
        APRNET_STORE_WEIGHTS()
        __syncthreads();
        if (ci0 + CIB < a.Cin) {
            load_items<G, float, CIB>(a, ci0 + CIB, nitem, tree_items, sh, R);
            APRNET_LOAD_WEIGHTS(ci0 / CIB + 1)
        }
#pragma unroll
        for (int p = 0; p < CIB / 2; ++p) {
#pragma unroll
            for (int t = 0; t < G::K; ++t) {
                const float av = ap[(2 * p * G::K + t) * WLD];
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const float bv = patch[bbase[j] + 2 * p * G::CH_STRIDE + tap_offset<G>(t)];
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[j], 0, 0, 0);
                }
            }
        }
    }
#undef APRNET_LOAD_WEIGHTS
#undef APRNET_STORE_WEIGHTS
    // D layout: lane l, register r -> column l%32, row 8*(r/4) + 4*(l/32) + r%4
    if constexpr (MODE == 0) {
        float bias[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) bias[r] = bias_l[8 * (r >> 2) + 4 * (lane >> 5) + (r & 3)];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 5) + (lane & 31);
            if (col >= nc) continue;
            const int64_t o = sh.col_idx[col];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int co = co0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (co < a.Cout) a.y[(int64_t)co * a.ldy + o] = acc[j][r] + bias[r];
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 5) + (lane & 31);
            if (col >= nc) continue;
            const bool to_tree = (sh.col_pos[col] & COL_TREE) != 0;
            float* dst = (to_tree ? a.gtree : a.gx) + sh.col_idx[col];
            const int64_t ld = to_tree ? a.ldgt : a.ldgx;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int ci = co0 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (ci < a.Cout) unsafeAtomicAdd(dst + (int64_t)ci * ld, acc[j][r]);
            }
        }
    }
}

template <class G, int CIB, int NBW, int MODE>
__global__ void __launch_bounds__(G::NT)
conv_mfma_kernel(const ConvArgs<float> a) {
    static_assert(CIB % 2 == 0, "input channels are consumed in pairs");
    static_assert((G::NWAVE & (G::NWAVE - 1)) == 0, "block rotation assumes a power-of-two wave count");
    static_assert(NBW == 2 && (G::MAXCOL + 31) / 32 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    __shared__ float patch[CIB * G::CH_STRIDE];
    __shared__ __attribute__((aligned(16))) float Wl[CIB * G::K * 32];
    __shared__ ConvShared<G> sh;
    __shared__ __attribute__((aligned(16))) float bias_l[32];   // bias of this block's output channels (0 without bias)

    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level, z0 = tile.z0, x0 = tile.x0;
    const int co0 = blockIdx.y * 32;
    const int yn = a.apr.y_num[L];
    const int s_idx = min(a.S_exp - 1, a.Lc - L);
    const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
    // packed weights of this level and block of 32 output channels: [chunk][CIB*K][32]
    const int nq = (a.Cin + CIB - 1) / CIB;
    const float4* __restrict__ wl = reinterpret_cast<const float4*>(a.w) +
                                    ((int64_t)s_idx * gridDim.y + blockIdx.y) * nq * (CIB * G::K * 8);
    const int wave = threadIdx.x >> 6;

    if (MODE == 0 && threadIdx.x < 32)
        bias_l[threadIdx.x] = (a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;
    open_segments<G, float>(a, L, z0, x0, sh);
    __syncthreads();

    int win = 0;
    for (int y0 = 0; y0 < yn; y0 += G::TY, ++win) {
        if constexpr (MODE == 0) scan_window<G, float>(a, L, y0, out_tree, sh);
        else scan_window_dx<G, float>(a, L, y0, out_tree, sh);
        __syncthreads();
        const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
        const bool tree_items = MODE == 0 && L < a.Lc;       // the output gradient has no tree part
        if (nc > 0 && nitem > 0) {
            const int nblk = (nc + 31) >> 5;
            // rotation: spread the waves that own one block more over the SIMDs
            const int first = (wave - (int)blockIdx.x - win) & (G::NWAVE - 1);
            const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;
            switch (__builtin_amdgcn_readfirstlane(nb)) {
                case 0: mfma_window<G, CIB, 0, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 1: mfma_window<G, CIB, 1, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                default: mfma_window<G, CIB, 2, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
            }
        }
        __syncthreads();
        close_window<G>(sh);
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------------------------------------
// Layers with at most 16 output channels: v_mfma_f32_16x16x4_f32, M = 16 output channels, N = 16 columns,
// K = the four input channels of a chunk at one tap.
//     A: lane l -> W[co = l%16][ci = l/16]      B: lane l -> patch[ci = l/16][cell of column l%16 + off(t)]
//     D: lane l, register r -> column l%16, output channel 4*(l/16) + r
// Half the matrix work of the 32-row kernel for these layers; a wave owns up to four blocks of 16 columns.
typedef float floatx4 __attribute__((ext_vector_type(4)));

// packed16[s][cb][q][t][c][16 co]: the chunk image is linear in (t, lane)
__global__ void pack_weights16_kernel(const float* __restrict__ w, int S_exp, int Cout, int Cin, int K, int CIB,
                                      float* __restrict__ out) {
    const int ncb = (Cout + 15) / 16, nq = (Cin + CIB - 1) / CIB;
    const int64_t n = (int64_t)S_exp * ncb * nq * K * CIB * 16;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        const int co = (int)(e % 16);
        const int c = (int)((e / 16) % CIB);
        const int t = (int)((e / (16 * CIB)) % K);
        const int q = (int)((e / (16 * (int64_t)CIB * K)) % nq);
        const int cb = (int)((e / (16 * (int64_t)CIB * K * nq)) % ncb);
        const int s = (int)(e / (16 * (int64_t)CIB * K * nq * ncb));
        const int ci = q * CIB + c, cog = cb * 16 + co;
        out[e] = (ci < Cin && cog < Cout) ? w[(((int64_t)s * Cout + cog) * Cin + ci) * K + t] : 0.f;
    }
}

template <class G, int NB>
__device__ __forceinline__ void mfma16_window(const ConvArgs<float>& a, int co0, int nc, int nitem, bool tree_items, int first,
                                              const float4* __restrict__ wl, const ConvShared<G>& sh,
                                              float* __restrict__ patch, float* __restrict__ Wl,
                                              const float* __restrict__ bias_l) {
    constexpr int CIB = 4;
    constexpr int KC = CIB * G::K;             // k rows per chunk
    const int lane = lane_id();
    constexpr int NBA = NB > 0 ? NB : 1;
    int bbase[NBA];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
        const int pos = col < nc ? (int)(sh.col_pos[col] & COL_CELL) - G::TAP0 : 0;
        bbase[j] = pos + (lane >> 4) * G::CH_STRIDE;
    }
    floatx4 acc[NBA];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[j][r] = 0.f;
    const float* ap = Wl + lane;

    constexpr int W4 = KC * 4;                                   // float4 elements of a weight chunk (16 co wide)
    constexpr int WPT = (W4 + G::NT - 1) / G::NT;
    ItemRegs<G, float, CIB> R;
    float4 wr[WPT];
#define APRNET_LOAD_WEIGHTS(q)                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        wr[k] = (i < W4) ? (wl + (int64_t)(q) * W4)[i] : make_float4(0.f, 0.f, 0.f, 0.f);          \
    }
#define APRNET_STORE_WEIGHTS()                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        if (i < W4) reinterpret_cast<float4*>(Wl)[i] = wr[k];                                      \
    }
    load_items<G, float, CIB>(a, 0, nitem, tree_items, sh, R);
    APRNET_LOAD_WEIGHTS(0)
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    for (int ci0 = 0; ci0 < a.Cin; ci0 += CIB) {
        __syncthreads();
        store_items<G, float, CIB>(R, nitem, patch);
        APRNET_STORE_WEIGHTS()
        __syncthreads();
        if (ci0 + CIB < a.Cin) {
            load_items<G, float, CIB>(a, ci0 + CIB, nitem, tree_items, sh, R);
            APRNET_LOAD_WEIGHTS(ci0 / CIB + 1)
        }
#pragma unroll
        for (int t = 0; t < G::K; ++t) {
            const float av = ap[t * 64];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const float bv = patch[bbase[j] + tap_offset<G>(t)];
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[j], 0, 0, 0);
            }
        }
    }
#undef APRNET_LOAD_WEIGHTS
#undef APRNET_STORE_WEIGHTS
    float bias[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) bias[r] = bias_l[4 * (lane >> 4) + r];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
        if (col >= nc) continue;
        const int64_t o = sh.col_idx[col];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int co = co0 + 4 * (lane >> 4) + r;
            if (co < a.Cout) a.y[(int64_t)co * a.ldy + o] = acc[j][r] + bias[r];
        }
    }
}

template <class G>
__global__ void __launch_bounds__(G::NT)
conv_mfma16_kernel(const ConvArgs<float> a) {
    constexpr int CIB = 4, NBW = 4;
    static_assert((G::NWAVE & (G::NWAVE - 1)) == 0, "block rotation assumes a power-of-two wave count");
    static_assert((G::MAXCOL + 15) / 16 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    static_assert(G::CH_STRIDE % 64 == 16, "four lane groups read four channels: a quarter of the banks each");
    __shared__ float patch[CIB * G::CH_STRIDE];
    __shared__ __attribute__((aligned(16))) float Wl[CIB * G::K * 16];
    __shared__ ConvShared<G> sh;
    __shared__ float bias_l[16];

    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level, z0 = tile.z0, x0 = tile.x0;
    const int co0 = blockIdx.y * 16;
    const int yn = a.apr.y_num[L];
    const int s_idx = min(a.S_exp - 1, a.Lc - L);
    const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
    const int nq = (a.Cin + CIB - 1) / CIB;
    const float4* __restrict__ wl = reinterpret_cast<const float4*>(a.w) +
                                    ((int64_t)s_idx * gridDim.y + blockIdx.y) * nq * (CIB * G::K * 4);
    const int wave = threadIdx.x >> 6;

    if (threadIdx.x < 16) bias_l[threadIdx.x] = (a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;
    open_segments<G, float>(a, L, z0, x0, sh);
    __syncthreads();

    int win = 0;
    for (int y0 = 0; y0 < yn; y0 += G::TY, ++win) {
        scan_window<G, float>(a, L, y0, out_tree, sh);
        __syncthreads();
        const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
        const bool tree_items = L < a.Lc;
        if (nc > 0) {
            const int nblk = (nc + 15) >> 4;
            const int first = (wave - (int)blockIdx.x - win) & (G::NWAVE - 1);
            const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;
            switch (__builtin_amdgcn_readfirstlane(nb)) {
                case 0: mfma16_window<G, 0>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 1: mfma16_window<G, 1>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 2: mfma16_window<G, 2>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 3: mfma16_window<G, 3>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                default: mfma16_window<G, 4>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
            }
        }
        __syncthreads();
        close_window<G>(sh);
        __syncthreads();
    }
}

using M333N = ConvGeom<3, 3, 3, 2, 4, 512, 64, 16>;

int launch_conv333_mfma16(const ConvArgs<float>& a, int n_tiles, hipStream_t st) {
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 15) / 16));
    hipLaunchKernelGGL((conv_mfma16_kernel<M333N>), grid, dim3(M333N::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma16_kernel");
    return 0;
}

size_t conv333_packed16_floats(int S_exp, int Cout, int Cin) {
    return (size_t)S_exp * ((Cout + 15) / 16) * ((Cin + 3) / 4) * 4 * 27 * 16;
}

int pack_conv333_weights16(const float* w, int S_exp, int Cout, int Cin, float* packed, hipStream_t st) {
    const size_t n = conv333_packed16_floats(S_exp, Cout, Cin);
    dim3 grid((unsigned)std::min<size_t>((n + 255) / 256, 2048));
    hipLaunchKernelGGL(pack_weights16_kernel, grid, dim3(256), 0, st, w, S_exp, Cout, Cin, 27, 4, packed);
    APRNET_LAUNCH_CHECK("pack_weights16_kernel");
    return 0;
}

using M333 = ConvGeom<3, 3, 3, 2, 4, 512>;

constexpr int MFMA_CIB = 4;

// a.w must point at the packed weights (pack_conv333_weights)
int launch_conv333_mfma(const ConvArgs<float>& a, int n_tiles, hipStream_t st) {
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 31) / 32));
    hipLaunchKernelGGL((conv_mfma_kernel<M333, MFMA_CIB, 2, 0>), grid, dim3(M333::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma_kernel (forward)");
    return 0;
}

// Input gradient: a.x / a.Cin describe the output gradient, a.Cout the input channels, a.w the packed
// transposed weights, a.tiles the row groups within one cell of an output (n_tiles of them).
int launch_conv333_dx_mfma(const ConvArgs<float>& a, int n_tiles, hipStream_t st) {
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 31) / 32));
    hipLaunchKernelGGL((conv_mfma_kernel<M333, MFMA_CIB, 2, 1>), grid, dim3(M333::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma_kernel (input gradient)");
    return 0;
}

// Cm: channels on the M axis of the kernel, Ck: contracted channels (forward: Cout, Cin; transposed: Cin, Cout)
size_t conv333_packed_floats(int S_exp, int Cm, int Ck) {
    return (size_t)S_exp * ((Cm + 31) / 32) * ((Ck + MFMA_CIB - 1) / MFMA_CIB) * MFMA_CIB * 27 * 32;
}

int pack_conv333_weights(const float* w, int S_exp, int Cm, int Ck, bool transposed, float* packed, hipStream_t st) {
    const size_t n = conv333_packed_floats(S_exp, Cm, Ck);
    dim3 grid((unsigned)std::min<size_t>((n + 255) / 256, 2048));
    hipLaunchKernelGGL(pack_weights_kernel, grid, dim3(256), 0, st, w, S_exp, Cm, Ck, 27, MFMA_CIB, transposed ? 1 : 0, packed);
    APRNET_LAUNCH_CHECK("pack_weights_kernel");
    return 0;
}

}  // namespace aprnet
