// Stencil convolution on the matrix cores (fp32 MFMA), gfx950: forward, and the gradient of the input.
//
// Same tiles, windows and three-source LDS gather as the VALU path (conv_common.hpp); only the
// contraction differs.  For one window the block holds nc output positions ("columns").  The
// contraction  out[co][col] = sum_{ci,t} W[co][ci][t] * patch[ci][pos(col) + off(t)]  is an implicit
// GEMM with M = output channels, N = columns, K = (tap, input channel).  Every lane owns one column and
// one channel of the staged chunk: its B operand for tap t sits at a fixed per-lane LDS address plus a
// compile-time tap offset, and its A operand at (t, lane) of a weight chunk that is re-laid out once per
// call so that staging it is a straight 16-byte copy.  The K loop is fully unrolled: ds_read_b32 with
// immediate offsets and MFMAs, no address arithmetic.  A wave keeps the accumulators of its column blocks
// in registers across all channel chunks, so each output element is written once (forward: no atomics,
// deterministic).
//
// The gradient of the input runs the same kernel on the output gradient with the transposed, flipped
// stencil (scan_window_dx in conv_common.hpp) and adds its results atomically.
//
// fp32 MFMA shares the SIMD's vector ALU on this hardware: while a wave's MFMA executes, no other wave of
// that SIMD issues vector instructions, and switching between the two costs a pipeline bubble.  The
// staging code therefore keeps its vector-instruction count low and the MFMA phases long.
#include "conv_common.hpp"

namespace aprnet {

template <class G>
__device__ __forceinline__ constexpr int tap_offset(int t) {
    return ((t / (G::KX * G::KY)) * G::RX + (t / G::KY) % G::KX) * G::RS + (t % G::KY);
}

// ---------------------------------------------------------------------------------------------------------
// The contraction: v_mfma_f32_16x16x4_f32, M = 16 output channels, N = 16 columns, K = the four input
// channels of a chunk at one tap.
//     A: lane l -> W[co = l%16][ci = l/16]      B: lane l -> patch[ci = l/16][cell of column l%16 + off(t)]
//     D: lane l, register r -> column l%16, output channel 4*(l/16) + r
// An output block holds COH parts of 16 channels (1 for layers of at most 16 outputs, else 2) that share
// the B operand; a wave owns up to four blocks of 16 columns.  Blocks of 16 columns instead of 32 waste
// less of the last block of a window and spread more evenly over the four SIMDs.
typedef float floatx4 __attribute__((ext_vector_type(4)));

// packed16[s][cb][q][t][h][c][16 co], cb = block of 16 * COH output channels, h = its 16-channel part:
// the chunk image is linear in (t, h, lane)
// With `transposed` the roles of the two channel axes are swapped and the taps reversed: the image is that
// of the stencil of the input gradient, M = input channels, contraction over (flipped tap, output channel).
// Cm / Ck are the channel counts of the M axis and of the contracted axis.
__global__ void pack_weights16_kernel(const float* __restrict__ w, int S_exp, int Cm, int Ck, int K, int CIB, int COH,
                                      int transposed, float* __restrict__ out) {
    const int Cout = transposed ? Ck : Cm, Cin = transposed ? Cm : Ck;
    const int ncb = (Cm + 16 * COH - 1) / (16 * COH), nq = (Ck + CIB - 1) / CIB;
    const int64_t n = (int64_t)S_exp * ncb * nq * K * COH * CIB * 16;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = e;
        const int co = (int)(r % 16); r /= 16;
        const int c = (int)(r % CIB); r /= CIB;
        const int h = (int)(r % COH); r /= COH;
        const int t = (int)(r % K); r /= K;
        const int q = (int)(r % nq); r /= nq;
        const int cb = (int)(r % ncb); r /= ncb;
        const int s = (int)r;
        const int ck = q * CIB + c, cm = (cb * COH + h) * 16 + co;
        float v = 0.f;
        if (ck < Ck && cm < Cm)
            v = transposed ? w[(((int64_t)s * Cout + ck) * Cin + cm) * K + (K - 1 - t)]
                           : w[(((int64_t)s * Cout + cm) * Cin + ck) * K + t];
        out[e] = v;
    }
}

// MODE 0: forward, results stored (plus bias).  MODE 1: input gradient, results added atomically to the
// place each column names (feature gradient, or tree gradient with COL_TREE).
template <typename T, class G, int COH, int NB, int MODE>
__device__ __forceinline__ void mfma16_window(const ConvArgs<T>& a, int co0, int nc, int nitem, bool tree_items, int first,
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
    floatx4 acc[NBA][COH];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int h = 0; h < COH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][h][r] = 0.f;
    const float* ap = Wl + lane;

    constexpr int W4 = KC * 4 * COH;                             // float4 elements of a weight chunk
    constexpr int WPT = (W4 + G::NT - 1) / G::NT;
    ItemRegs<G, T, CIB> R;
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
    load_items<G, T, CIB>(a, 0, nitem, tree_items, sh, R);
    APRNET_LOAD_WEIGHTS(0)
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    for (int ci0 = 0; ci0 < a.Cin; ci0 += CIB) {
        __syncthreads();
        store_items<G, T, CIB>(R, nitem, patch);
        APRNET_STORE_WEIGHTS()
        __syncthreads();
        if (ci0 + CIB < a.Cin) {
            load_items<G, T, CIB>(a, ci0 + CIB, nitem, tree_items, sh, R);
            APRNET_LOAD_WEIGHTS(ci0 / CIB + 1)
        }
#pragma unroll
        for (int t = 0; t < G::K; ++t) {
            float av[COH];
#pragma unroll
            for (int h = 0; h < COH; ++h) av[h] = ap[(t * COH + h) * 64];
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const float bv = patch[bbase[j] + tap_offset<G>(t)];
#pragma unroll
                for (int h = 0; h < COH; ++h) acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[h], bv, acc[j][h], 0, 0, 0);
            }
        }
    }
#undef APRNET_LOAD_WEIGHTS
#undef APRNET_STORE_WEIGHTS
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
        if (col >= nc) continue;
        const int64_t o = sh.col_idx[col];
        if constexpr (MODE == 0) {
#pragma unroll
            for (int h = 0; h < COH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int cl = h * 16 + 4 * (lane >> 4) + r;
                    if (co0 + cl < a.Cout) a.y[(int64_t)(co0 + cl) * a.ldy + o] = Num<T>::st(acc[j][h][r] + bias_l[cl]);
                }
        } else if constexpr (sizeof(T) == 4) {      // gradients are accumulated in fp32 only
            const bool to_tree = (sh.col_pos[col] & COL_TREE) != 0;
            float* dst = (to_tree ? a.gtree : a.gx) + o;
            const int64_t ld = to_tree ? a.ldgt : a.ldgx;
#pragma unroll
            for (int h = 0; h < COH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int cl = h * 16 + 4 * (lane >> 4) + r;
                    if (co0 + cl < a.Cout) unsafeAtomicAdd(dst + (int64_t)(co0 + cl) * ld, acc[j][h][r]);
                }
        }
    }
}

// COH = 16-channel parts of the output block: 1 for layers of at most 16 output channels, 2 otherwise
// Three workgroups per CU (six waves per SIMD, 80 registers): the third group hides more of the latency of
// the scan and staging phases than the few spilled registers cost.
template <typename T, class G, int COH, int MODE>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(6, 6)))
conv_mfma16_kernel(const ConvArgs<T> a) {
    constexpr int CIB = 4, NBW = 4;
    static_assert((G::NWAVE & (G::NWAVE - 1)) == 0, "block rotation assumes a power-of-two wave count");
    static_assert((G::MAXCOL + 15) / 16 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    static_assert(G::CH_STRIDE % 64 == 16, "four lane groups read four channels: a quarter of the banks each");
    __shared__ float patch[CIB * G::CH_STRIDE];
    __shared__ __attribute__((aligned(16))) float Wl[CIB * G::K * 16 * COH];
    __shared__ ConvShared<G> sh;
    __shared__ float bias_l[16 * COH];

    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level, z0 = tile.z0, x0 = tile.x0;
    const int co0 = blockIdx.y * 16 * COH;
    const int yn = a.apr.y_num[L];
    const int s_idx = min(a.S_exp - 1, a.Lc - L);
    const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
    const int nq = (a.Cin + CIB - 1) / CIB;
    const float4* __restrict__ wl = reinterpret_cast<const float4*>(a.w) +
                                    ((int64_t)s_idx * gridDim.y + blockIdx.y) * nq * (CIB * G::K * 4 * COH);
    const int wave = threadIdx.x >> 6;

    if (MODE == 0 && threadIdx.x < 16 * COH)
        bias_l[threadIdx.x] = (a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;
    open_segments<G, T>(a, L, z0, x0, sh);
    __syncthreads();

    int win = 0;
    for (int y0 = 0; y0 < yn; y0 += G::TY, ++win) {
        if constexpr (MODE == 0) scan_window<G, T>(a, L, y0, out_tree, sh);
        else scan_window_dx<G, T>(a, L, y0, out_tree, sh);
        __syncthreads();
        const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
        const bool tree_items = MODE == 0 && L < a.Lc;       // the output gradient has no tree part
        if (nc > 0 && nitem > 0) {
            const int nblk = (nc + 15) >> 4;
            const int first = (wave - (int)blockIdx.x - win) & (G::NWAVE - 1);
            const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;
            switch (__builtin_amdgcn_readfirstlane(nb)) {
                case 0: mfma16_window<T, G, COH, 0, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 1: mfma16_window<T, G, COH, 1, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 2: mfma16_window<T, G, COH, 2, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                case 3: mfma16_window<T, G, COH, 3, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
                default: mfma16_window<T, G, COH, 4, MODE>(a, co0, nc, nitem, tree_items, first, wl, sh, patch, Wl, bias_l); break;
            }
        }
        __syncthreads();
        close_window<G>(sh);
        __syncthreads();
    }
}

using M333N = ConvGeom<3, 3, 3, 2, 4, 512, 64, 16>;
using M133N = ConvGeom<1, 3, 3, 1, 8, 512, 64, 16>;
using M155N = ConvGeom<1, 5, 5, 1, 8, 512, 64, 16>;

// stencils with a matrix-core kernel (kz*100 + kx*10 + ky); 5x5x5 needs a weight chunk that does not fit LDS
bool conv_mfma_supported(int code) { return code == 333 || code == 133 || code == 155; }
static int conv_taps(int code) { return code == 333 ? 27 : code == 133 ? 9 : 25; }
static int conv_coh(int Cm) { return Cm <= 16 ? 1 : 2; }

template <typename T, class G, int MODE>
static int launch16(const ConvArgs<T>& a, int n_tiles, hipStream_t st) {
    const int coh = conv_coh(a.Cout);
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 16 * coh - 1) / (16 * coh)));
    if (coh == 1) hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 1, MODE>), grid, dim3(G::NT), 0, st, a);
    else hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 2, MODE>), grid, dim3(G::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma16_kernel");
    return 0;
}
template <typename T, int MODE>
static int launch16_code(int code, const ConvArgs<T>& a, int n_tiles, hipStream_t st) {
    switch (code) {
        case 333: return launch16<T, M333N, MODE>(a, n_tiles, st);
        case 133: return launch16<T, M133N, MODE>(a, n_tiles, st);
        case 155: return launch16<T, M155N, MODE>(a, n_tiles, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "no matrix-core kernel for this stencil");
}

// Forward.  a.w must point at the packed weights (pack_conv_weights).
int launch_conv_mfma(int code, const ConvArgs<float>& a, int n_tiles, hipStream_t st) { return launch16_code<float, 0>(code, a, n_tiles, st); }
int launch_conv_mfma(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st) { return launch16_code<bf16_t, 0>(code, a, n_tiles, st); }

// Input gradient: a.x / a.Cin describe the output gradient, a.Cout the input channels, a.w the packed
// transposed weights, a.tiles the row groups within one row of an output (n_tiles of them).
int launch_conv_dx_mfma(int code, const ConvArgs<float>& a, int n_tiles, hipStream_t st) { return launch16_code<float, 1>(code, a, n_tiles, st); }

// Cm: channels on the M axis of the kernel, Ck: contracted channels (forward: Cout, Cin; transposed: Cin, Cout)
size_t conv_packed_floats(int code, int S_exp, int Cm, int Ck) {
    const int coh = conv_coh(Cm);
    return (size_t)S_exp * ((Cm + 16 * coh - 1) / (16 * coh)) * ((Ck + 3) / 4) * 4 * conv_taps(code) * 16 * coh;
}

int pack_conv_weights(int code, const float* w, int S_exp, int Cm, int Ck, bool transposed, float* packed, hipStream_t st) {
    const size_t n = conv_packed_floats(code, S_exp, Cm, Ck);
    dim3 grid((unsigned)std::min<size_t>((n + 255) / 256, 2048));
    hipLaunchKernelGGL(pack_weights16_kernel, grid, dim3(256), 0, st, w, S_exp, Cm, Ck, conv_taps(code), 4, conv_coh(Cm),
                       transposed ? 1 : 0, packed);
    APRNET_LAUNCH_CHECK("pack_weights16_kernel");
    return 0;
}

}  // namespace aprnet
