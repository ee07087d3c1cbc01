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

typedef int intx4w __attribute__((ext_vector_type(4)));

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
// Input channels per staged chunk (a multiple of the 4 of one instruction) and waves per SIMD the kernels are
// compiled for.  Three workgroups per CU (six waves per SIMD, 80 registers) beat two with chunks of 8: the
// third group hides more of the latency between the matrix phases than the few spilled registers cost.
// Forward takes its window lists from the plan; the input gradient scans and keeps its lists in LDS.
// (Layers of at most 16 outputs fit 64 registers without spilling; four workgroups per CU instead of three make the
// plain 16->16 layer 2 % faster, 4.29 -> 4.21 ms, and the network, whose 16-output layers are the fused forms, 0.8 % slower.)
constexpr int FWD_CIB = 4, FWD_WAVES = 6;
constexpr int DX_CIB = 4, DX_WAVES = 6;
constexpr int STAGE_PRIO = 3;      // wave priority outside the matrix loops

// packed16[s][cb][q][t][h][c][16 co], cb = block of 16 * COH output channels, h = its 16-channel part:
// the chunk image is linear in (t, h, lane)
// With `transposed` the roles of the two channel axes are swapped and the taps reversed: the image is that
// of the stencil of the input gradient, M = input channels, contraction over (flipped tap, output channel).
// Cm / Ck are the channel counts of the M axis and of the contracted axis.
__global__ void pack_weights16_kernel(const float* __restrict__ w, int S_exp, int Cm, int Ck, int K, int CIB, int COH,
                                      int transposed, float* __restrict__ out) {
    const int Cout = transposed ? Ck : Cm, Cin = transposed ? Cm : Ck;
    const int ncb = (Cm + 16 * COH - 1) / (16 * COH), nq = (Ck + CIB - 1) / CIB;
    // 32-bit index arithmetic (the host checks that the image has fewer than 2^31 elements): 64-bit divisions made
    // this tiny kernel take longer than the convolution of a coarse level
    const unsigned n = (unsigned)S_exp * ncb * nq * K * COH * CIB * 16;
    for (unsigned e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        unsigned r = e;
        const int co = (int)(r % 16u); r /= 16u;
        const int c = (int)(r % (unsigned)CIB); r /= (unsigned)CIB;
        const int h = (int)(r % (unsigned)COH); r /= (unsigned)COH;
        const int t = (int)(r % (unsigned)K); r /= (unsigned)K;
        const int q = (int)(r % (unsigned)nq); r /= (unsigned)nq;
        const int cb = (int)(r % (unsigned)ncb); r /= (unsigned)ncb;
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
template <typename T, class G, int CIB, int COH, int NB, int MODE, bool FUSE, class Lists>
__device__ __forceinline__ void mfma16_window(const ConvArgs<T>& a, int co0, int nc, int nitem, bool tree_items, int first,
                                              const float4* __restrict__ wl, const Lists& sh,
                                              float* __restrict__ patch, float* __restrict__ Wl,
                                              const float* __restrict__ bias_l) {
    constexpr int NSUB = CIB / 4;
    constexpr int KC = CIB * G::K;             // k rows per chunk
    const int lane = lane_id();
    constexpr int NBA = NB > 0 ? NB : 1;
    int bbase[NBA];
    constexpr bool LISTED = std::is_same<Lists, WindowLists>::value;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
        unsigned cp;
        if constexpr (LISTED) {
            // lists in global memory: an unconditional load (columns past the end read zero), so that it travels with the
            // slot loads below instead of being waited for on the spot, as a load under `col < nc` is
            const __amdgpu_buffer_rsrc_t rcp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(sh.col_pos), 0, nc * 2, 0x00020000);
            cp = (unsigned)__builtin_amdgcn_raw_buffer_load_b16(rcp, col * 2, 0, 0) & 0xffffu;
            bbase[j] = (int)cp;
        } else {
            cp = col < nc ? (unsigned)sh.col_pos[col] : (unsigned)G::TAP0;
            // pooled columns of the input gradient read the box-summed patch that follows the patch in LDS
            bbase[j] = (int)(cp & COL_CELL) - G::TAP0 + (lane >> 4) * G::CH_STRIDE + ((MODE == 1 && (cp & COL_BOX)) ? CIB * G::CH_STRIDE : 0);
        }
    }
    floatx4 acc[NBA][COH];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int h = 0; h < COH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][h][r] = 0.f;
    const float* ap = Wl + lane;
    // B operands are read through a volatile LDS pointer: that keeps them single ds_read_b32 with immediate
    // offsets.  Paired into ds_read2 they need vector adds for their bases inside the matrix loop, and a vector
    // instruction between two MFMAs costs a pipeline switch; it also keeps the loop within 80 registers.
    typedef const volatile __attribute__((address_space(3))) float lds_float;
    lds_float* lpatch = (lds_float*)patch;

    constexpr int W4 = KC * 4 * COH;                             // float4 elements of a weight chunk
    constexpr int WPT = (W4 + G::NT - 1) / G::NT;
    ItemRegs<G, T, CIB> R;
    // The weights of a chunk come through unconditional buffer loads (lanes past the end read zeros): under a
    // per-lane branch the compiler waits for every load in flight before it enters the branch, which made each
    // chunk wait for the feature loads issued just before instead of letting them travel during the matrix phase.
    intx4w wr[WPT];
#define APRNET_LOAD_WEIGHTS(q)                                                                     \
    {                                                                                              \
        const __amdgpu_buffer_rsrc_t rw_ = __builtin_amdgcn_make_buffer_rsrc(                      \
            const_cast<float4*>(wl + (int64_t)(q) * W4), 0, W4 * 16, 0x00020000);                  \
        _Pragma("unroll") for (int k = 0; k < WPT; ++k)                                            \
            wr[k] = __builtin_amdgcn_raw_buffer_load_b128(rw_, (int)(threadIdx.x + k * G::NT) * 16, 0, 0); \
    }
#define APRNET_STORE_WEIGHTS()                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        if (i < W4) reinterpret_cast<intx4w*>(Wl)[i] = wr[k];                                      \
    }
    // Staging runs at a raised wave priority, the matrix loop at the default one: fp32 matrix instructions share the
    // SIMD's vector pipe, and a workgroup that is staging gets back to its own matrix phase sooner when its few
    // vector instructions are not queued behind the other workgroups' matrix loops (15.0 -> 14.8 ms).
    __builtin_amdgcn_s_setprio(STAGE_PRIO);
    load_items<G, T, CIB>(a, 0, nitem, tree_items, sh, R, 0, std::bool_constant<FUSE>{});
    if constexpr (LISTED) {
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            const unsigned cp = col < nc ? (unsigned)bbase[j] : (unsigned)G::TAP0;
            bbase[j] = (int)(cp & COL_CELL) - G::TAP0 + (lane >> 4) * G::CH_STRIDE + ((MODE == 1 && (cp & COL_BOX)) ? CIB * G::CH_STRIDE : 0);
        }
    }
    APRNET_LOAD_WEIGHTS(0)
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    for (int ci0 = 0; ci0 < a.Cin; ci0 += CIB) {
        __syncthreads();
        store_items<G, T, CIB>(R, nitem, patch);
        APRNET_STORE_WEIGHTS()
        __syncthreads();
        if (ci0 + CIB < a.Cin) {
            load_values<G, T, CIB>(a, ci0 + CIB, nitem, tree_items, R, 0, std::bool_constant<FUSE>{});
            APRNET_LOAD_WEIGHTS(ci0 / CIB + 1)
        }
        if constexpr (MODE == 1) {
            // Box sums over the cells of a coarser particle, for the pooled columns.  One wave per task
            // (channel, pair of z rows, part of the x range), one lane per y: the sums over y and z of every x
            // row are formed in registers, neighbouring x rows added, so each cell is read once per task.
            if (sh.nbox > 0) {
                constexpr int BOXZ = G::TZ >= 2 ? 2 : 1;
                constexpr int NZP = G::RZ - (BOXZ - 1);                 // first z rows of a box
                constexpr int XP = BOXZ == 1 ? 2 : 1, XW = (G::RX - 1 + XP - 1) / XP;      // x rows of boxes per task
                float* box = patch + CIB * G::CH_STRIDE;
                for (int task = threadIdx.x >> 6; task < CIB * NZP * XP; task += G::NWAVE) {
                    const int c = task / (NZP * XP), zp = (task / XP) % NZP, xb = (task % XP) * XW;
                    const float* p = patch + c * G::CH_STRIDE + (zp * G::RX + xb) * G::RS + lane;
                    float* q = box + c * G::CH_STRIDE + (zp * G::RX + xb) * G::RS + lane;
                    if (lane < G::RS - 1 && lane < 63) {
                        float prev = 0.f;
#pragma unroll
                        for (int x = 0; x <= XW; ++x) {
                            if (xb + x >= G::RX) break;
                            float s = p[x * G::RS] + p[x * G::RS + 1];
                            if (BOXZ == 2) s += p[(G::RX + x) * G::RS] + p[(G::RX + x) * G::RS + 1];
                            if (x > 0) q[(x - 1) * G::RS] = prev + s;
                            prev = s;
                        }
                    }
                }
                __syncthreads();
            }
        }
        __builtin_amdgcn_s_setprio(0);
        // The B operand of the next block is read before the matrix instructions of this one are issued, so that a
        // wave alone in its matrix phase does not sit out an LDS round trip per pair of instructions.
        if constexpr (NB > 0) {
            float bvn = lpatch[bbase[0] + tap_offset<G>(0)];
#pragma unroll
            for (int t = 0; t < G::K; ++t) {
#pragma unroll
                for (int sb = 0; sb < NSUB; ++sb) {
                    float av[COH];
#pragma unroll
                    for (int h = 0; h < COH; ++h) av[h] = ap[((t * COH + h) * NSUB + sb) * 64];
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const float bv = bvn;
                        if (j + 1 < NB) bvn = lpatch[bbase[j + 1] + 4 * sb * G::CH_STRIDE + tap_offset<G>(t)];
                        else if (sb + 1 < NSUB) bvn = lpatch[bbase[0] + 4 * (sb + 1) * G::CH_STRIDE + tap_offset<G>(t)];
                        else if (t + 1 < G::K) bvn = lpatch[bbase[0] + tap_offset<G>(t + 1 < G::K ? t + 1 : t)];
#pragma unroll
                        for (int h = 0; h < COH; ++h) acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[h], bv, acc[j][h], 0, 0, 0);
                    }
                }
            }
        }
        __builtin_amdgcn_s_setprio(STAGE_PRIO);
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
                    float v = acc[j][h][r] + bias_l[cl];
                    if (FUSE && a.relu) v = v < 0.f ? 0.f : v;
                    if (co0 + cl < a.Cout) a.y[(int64_t)(co0 + cl) * a.ldy + o] = Num<T>::st(v);
                }
        } else {
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
// LISTS: the windows of the tile come as precomputed lists from the plan (forward); otherwise the block scans
// the access arrays itself (input gradient).
// FUSE: built for the fused forward entry points (second input tensor, clamp at zero)
template <typename T, class G, int COH, int MODE, bool LISTS, bool FUSE = false>
__global__ void __launch_bounds__(G::NT)
__attribute__((amdgpu_waves_per_eu(LISTS ? FWD_WAVES : DX_WAVES, LISTS ? FWD_WAVES : DX_WAVES)))
conv_mfma16_kernel(const ConvArgs<T> a) {
    constexpr int CIB = LISTS ? FWD_CIB : DX_CIB, NBW = 4;
    static_assert((G::MAXCOL + 15) / 16 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    static_assert(G::CH_STRIDE % 64 == 16, "four lane groups read four channels: a quarter of the banks each");
    __shared__ float patch[(MODE == 1 ? 2 : 1) * CIB * G::CH_STRIDE];      // input gradient: patch + box sums
    __shared__ __attribute__((aligned(16))) float Wl[CIB * G::K * 16 * COH];
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
    const bool tree_items = MODE == 0 && L < a.Lc;       // the output gradient has no tree part

    if (MODE == 0 && threadIdx.x < 16 * COH)
        bias_l[threadIdx.x] = (a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;

#define APRNET_WINDOW(LISTS_OBJ)                                                                                          \
    {                                                                                                                     \
        const int nblk = (nc + 15) >> 4;                                                                                  \
        /* rotation: spread the waves that own one block more over the SIMDs */                                           \
        const int first = (wave + G::NWAVE - (int)((blockIdx.x + win) % G::NWAVE)) % G::NWAVE;                            \
        const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;                                       \
        switch (__builtin_amdgcn_readfirstlane(nb)) {                                                                     \
            case 0: mfma16_window<T, G, CIB, COH, 0, MODE, FUSE>(a, co0, nc, nitem, tree_items, first, wl, LISTS_OBJ, patch, Wl, bias_l); break; \
            case 1: mfma16_window<T, G, CIB, COH, 1, MODE, FUSE>(a, co0, nc, nitem, tree_items, first, wl, LISTS_OBJ, patch, Wl, bias_l); break; \
            case 2: mfma16_window<T, G, CIB, COH, 2, MODE, FUSE>(a, co0, nc, nitem, tree_items, first, wl, LISTS_OBJ, patch, Wl, bias_l); break; \
            case 3: mfma16_window<T, G, CIB, COH, 3, MODE, FUSE>(a, co0, nc, nitem, tree_items, first, wl, LISTS_OBJ, patch, Wl, bias_l); break; \
            default: mfma16_window<T, G, CIB, COH, 4, MODE, FUSE>(a, co0, nc, nitem, tree_items, first, wl, LISTS_OBJ, patch, Wl, bias_l); break; \
        }                                                                                                                 \
    }

    if constexpr (LISTS) {
        (void)z0; (void)x0; (void)yn; (void)out_tree;
        __shared__ int4 hdr[16];              // headers of sixteen windows: one round trip instead of one per window
        const int wb = a.tile_win[blockIdx.x], we = a.tile_win[blockIdx.x + 1];
        for (int w = wb; w < we; ++w) {
            const int win = w - wb;
            if ((win & 15) == 0) {            // every wave is past the previous window's last barrier
                if (threadIdx.x < 16 && w + (int)threadIdx.x < we) hdr[threadIdx.x] = a.win[w + threadIdx.x];
                __syncthreads();
            }
            const int4 hd = hdr[win & 15];
            const int nitem = __builtin_amdgcn_readfirstlane(hd.y), nc = __builtin_amdgcn_readfirstlane(hd.w);
            const unsigned i0 = (unsigned)__builtin_amdgcn_readfirstlane(hd.x), c0 = (unsigned)__builtin_amdgcn_readfirstlane(hd.z);
            const WindowLists gl{a.l_item_idx + i0, a.l_item_pos + i0, a.l_col_idx + c0, a.l_col_pos + c0};
            APRNET_WINDOW(gl)
            __syncthreads();        // the next window rewrites the patch
        }
    } else {
        __shared__ ConvShared<G> sh;
        open_segments<G, T>(a, L, z0, x0, sh);
        __syncthreads();
        int win = 0;
        for (int y0 = 0; y0 < yn; y0 += G::TY, ++win) {
            if constexpr (MODE == 0) scan_window<G, T>(a, L, y0, out_tree, sh);
            else scan_window_dx<G, T>(a, L, z0, x0, y0, out_tree, sh);
            __syncthreads();
            const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
            if (nc > 0 && nitem > 0) APRNET_WINDOW(sh)
            __syncthreads();
            close_window<G>(sh);
            __syncthreads();
        }
    }
#undef APRNET_WINDOW
}

// ---------------------------------------------------------------------------------------------------------
// bfloat16 contraction (forward, bfloat16 features): v_mfma_f32_16x16x32_bf16 (gfx950), fp32 accumulation.
// The 32 k of one instruction are 4 taps x 8 input channels: lane group g = l/16 supplies the eight bfloat16
// (16 bytes) of tap 4*step + g, the whole 8-channel chunk of one patch cell.
//     patch16[cell]        16 bytes = the 8 channels of the chunk at one cell
//     Wl16[step][h][lane]  16 bytes = the A operand of that lane (weights rounded to bfloat16 when packed)
// The sixteen lanes of a group read sixteen consecutive cells (256 bytes, every LDS bank once).  Same lists, same D
// layout and epilogue as the fp32 kernel; a window needs a quarter of the channel chunks and 1/16 of the matrix
// instructions.  (The K = 16 form of older parts runs at half the rate here: 16 cycles for 8192 flop.)
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr int BF_CIB = 8;

template <class G> constexpr int bf16_steps() { return (G::K + 3) / 4; }
// word offset of tap t's cell from the column's first tap; taps past the stencil (zero weights) re-read tap 0
template <class G> __device__ __forceinline__ int tap_offset_rt(int t) {
    if (t >= G::K) t = 0;
    return ((t / (G::KX * G::KY)) * G::RX + (t / G::KY) % G::KX) * G::RS + t % G::KY;
}

// packedB[s][cb][q][step][h][lane] (16 bytes each), cb = block of 16 * COH output channels, q = chunk of 8 inputs
// With `transposed` the image is that of the input gradient's stencil: the channel axes swap roles (Cout then
// names the input channels of the layer, Cin its output channels) and the taps are reversed.
__global__ void pack_weights_bf16_kernel(const float* __restrict__ w, int S_exp, int Cout, int Cin, int K, int COH,
                                         int transposed, uint4* __restrict__ out) {
    const int ncb = (Cout + 16 * COH - 1) / (16 * COH), nq = (Cin + BF_CIB - 1) / BF_CIB, nstep = (K + 3) / 4;
    const int64_t n = (int64_t)S_exp * ncb * nq * nstep * COH * 64;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t r = e;
        const int lane = (int)(r % 64); r /= 64;
        const int h = (int)(r % COH); r /= COH;
        const int step = (int)(r % nstep); r /= nstep;
        const int q = (int)(r % nq); r /= nq;
        const int cb = (int)(r % ncb); r /= ncb;
        const int s = (int)r;
        const int g = lane >> 4, co = (cb * COH + h) * 16 + (lane & 15);
        const int t = 4 * step + g, ci0 = q * BF_CIB;
        unsigned v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float f = 0.f;
            if (t < K && co < Cout && ci0 + j < Cin)
                f = transposed ? w[(((int64_t)s * Cin + ci0 + j) * Cout + co) * K + (K - 1 - t)]
                               : w[(((int64_t)s * Cout + co) * Cin + ci0 + j) * K + t];
            v[j] = float_to_bf16(f).bits;
        }
        out[e] = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
    }
}

template <class G>
__device__ __forceinline__ void store_items_bf16(const ItemRegs<G, bf16_t, BF_CIB>& R, int nitem, uint4* __restrict__ patch16) {
#pragma unroll
    for (int k = 0; k < ItemRegs<G, bf16_t, BF_CIB>::IPT; ++k) {
        if (k * G::NT >= nitem) break;                  // wave-uniform
        if (R.pos[k] == 0xffffu) continue;
        uint4* cell = patch16 + (R.pos[k] & ITEM_CELL);
        const uint4 v = make_uint4((unsigned)R.v[k][0] | ((unsigned)R.v[k][1] << 16), (unsigned)R.v[k][2] | ((unsigned)R.v[k][3] << 16),
                                   (unsigned)R.v[k][4] | ((unsigned)R.v[k][5] << 16), (unsigned)R.v[k][6] | ((unsigned)R.v[k][7] << 16));
        cell[0] = v;
        if (R.pos[k] & ITEM_PAIR) cell[1] = v;
    }
}

// ---- regrouped input: [Cin / 8][count][8] bfloat16 -----------------------------------------------------------
// A sparse row inside a window holds few particles, so a gather of one 2-byte channel value per lane touches
// about twenty cache lines per wave and the kernel waits for memory two thirds of the time.  With the 8 channels
// of a group next to each other an item is ONE 16-byte load per round of staging instead of eight 2-byte loads
// through eight descriptors: an eighth of the load instructions, a quarter of the value registers, two
// descriptors instead of sixteen.  The regrouping is one streaming pass over the input (interleave8_kernel).
typedef int intx4 __attribute__((ext_vector_type(4)));
template <class G, int IPT>
struct ItemRegs16 { intx4 v[IPT]; unsigned off[IPT]; unsigned short pos[IPT]; };

// BIG: tensors of 2^28 elements and more per group, whose 16-byte items lie past 32-bit byte offsets: R.off keeps the
// element index and the loads take 64-bit addresses (a lane without an item reads element 0; its value is never stored)
template <class G, int IPT, bool BIG = false, class Lists>
__device__ __forceinline__ void fetch_slots16(const Lists& sh, int nitem, ItemRegs16<G, IPT>& R) {
    // unconditional buffer loads, results touched only after every round is issued (see fetch_slots)
    const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(sh.item_idx), 0, nitem * 4, 0x00020000);
    const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(sh.item_pos), 0, nitem * 2, 0x00020000);
    int idx[IPT], pos[IPT];
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));                       // offsets formed per call, not kept (and spilled) across the window loop
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
        idx[k] = 0; pos[k] = 0;
        if (k * G::NT >= nitem) continue;               // wave-uniform
        const int it = tid + k * G::NT;
        idx[k] = __builtin_amdgcn_raw_buffer_load_b32(ri, it * 4, 0, 0);
        pos[k] = (int)__builtin_amdgcn_raw_buffer_load_b16(rp, it * 2, 0, 0);
    }
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
        const bool valid = (int)threadIdx.x + k * G::NT < nitem;
        R.pos[k] = valid ? (unsigned short)pos[k] : (unsigned short)0xffffu;
        R.off[k] = BIG ? (valid ? (unsigned)idx[k] : 0u) : (valid ? (unsigned)idx[k] * 16u : BUF_OOB);
    }
}
template <class G, int IPT, bool BIG = false>
__device__ __forceinline__ void load_values16(const ConvArgs<bf16_t>& a, int ci0, int nitem, bool tree_items, ItemRegs16<G, IPT>& R) {
    const int q = ci0 / BF_CIB;
    const int q1 = a.c_split / BF_CIB;          // groups of the first tensor when there is a second one
    const bf16_t* xg = (a.xi2 != nullptr && q >= q1) ? a.xi2 + (int64_t)(q - q1) * a.xi2_ld * BF_CIB : a.xi + (int64_t)q * a.xi_ld * BF_CIB;
    if constexpr (BIG) {
        const bf16_t* tg = a.ti + (int64_t)q * a.ti_ld * BF_CIB;
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            if (k * G::NT >= nitem) break;                  // wave-uniform
            const bool from_tree = tree_items && (R.pos[k] & ITEM_TREE) != 0 && R.pos[k] != 0xffffu;
            const bf16_t* base = from_tree ? tg : xg;       // a select, not a branch
            R.v[k] = *reinterpret_cast<const intx4*>(base + (uint64_t)R.off[k] * 8u);
        }
        return;
    }
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(xg), 0, (int)(a.x_count * 16), 0x00020000);
    const __amdgpu_buffer_rsrc_t rt = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(a.ti + (int64_t)q * a.ti_ld * BF_CIB), 0,
                                                                        tree_items ? (int)(a.t_count * 16) : 0, 0x00020000);
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
        if (k * G::NT >= nitem) break;                  // wave-uniform
        const bool from_tree = (R.pos[k] & ITEM_TREE) != 0 && R.pos[k] != 0xffffu;
        if (tree_items) {
            if (from_tree) {
                R.v[k] = __builtin_amdgcn_raw_buffer_load_b128(rt, (int)R.off[k], 0, 0);
                asm volatile("" ::: "memory");          // keeps the two branches from being merged into one load with a per-lane descriptor
            } else {
                R.v[k] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)R.off[k], 0, 0);
            }
        } else {
            R.v[k] = __builtin_amdgcn_raw_buffer_load_b128(rx, (int)R.off[k], 0, 0);
        }
    }
}
template <class G, int IPT>
__device__ __forceinline__ void store_items16(const ItemRegs16<G, IPT>& R, int nitem, uint4* __restrict__ patch16) {
#pragma unroll
    for (int k = 0; k < IPT; ++k) {
        if (k * G::NT >= nitem) break;                  // wave-uniform
        if (R.pos[k] == 0xffffu) continue;
        uint4* cell = patch16 + (R.pos[k] & ITEM_CELL);
        const uint4 v = make_uint4((unsigned)R.v[k][0], (unsigned)R.v[k][1], (unsigned)R.v[k][2], (unsigned)R.v[k][3]);
        cell[0] = v;
        if (R.pos[k] & ITEM_PAIR) cell[1] = v;
    }
}

// out[q][i][c] = channel 8 q + c of element i; channels from c_split on come from x2 (null: all from x), channels
// past C read as zeros.  One thread per (element, group): eight 2-byte reads along the planes, one 16-byte write.
__global__ void interleave8_kernel(const bf16_t* __restrict__ x, int64_t ldx, const bf16_t* __restrict__ x2, int64_t ldx2, int c_split,
                                   int C, int64_t count, bf16_t* __restrict__ out) {
    const int q = blockIdx.y;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x) {
        unsigned v[BF_CIB];
#pragma unroll
        for (int c = 0; c < BF_CIB; ++c) {
            const int ch = q * BF_CIB + c;
            v[c] = 0u;
            if (ch < C) v[c] = (x2 != nullptr && ch >= c_split) ? x2[(int64_t)(ch - c_split) * ldx2 + i].bits : x[(int64_t)ch * ldx + i].bits;
        }
        reinterpret_cast<uint4*>(out)[(int64_t)q * count + i] = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
    }
}

// MODE 0: forward.  MODE 1: input gradient (items = output gradient, results added atomically in fp32 to the place
// each column names, as in the fp32 kernel; no pooled columns).
// IL: the input comes regrouped (a.xi, a.ti), see above
// HEAD: the 1x1x1 convolution of the result follows here (see ConvArgs::head_w); head_a holds the A operands of the
// head's weights for this tile's level (per lane: bfloat16 heads, then bfloat16 remainders), head_b4 its bias
template <class G, int COH, int NB, bool FUSE, int MODE, bool IL, bool BIG, bool HEAD = false, class Lists>
__device__ __forceinline__ void mfma_bf16_window(const ConvArgs<bf16_t>& a, int co0, int nc, int nitem, bool tree_items, int first,
                                                 const uint4* __restrict__ wl, const Lists& sh,
                                                 uint4* __restrict__ patch16, uint4* __restrict__ Wl16,
                                                 const float* __restrict__ bias_l, const int* __restrict__ toff_l,
                                                 const uint4* __restrict__ head_a = nullptr, const float* __restrict__ head_b4 = nullptr) {
    constexpr int NSTEP = bf16_steps<G>();
    const int lane = lane_id();
    constexpr int NBA = NB > 0 ? NB : 1;
    int bbase[NBA], ocol[NBA];
    if constexpr (IL) {
        // cell and output index of this lane's columns: unconditional loads (columns past the end read zero) that
        // travel together with the list loads below instead of taking a round trip each
        const __amdgpu_buffer_rsrc_t rcp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(sh.col_pos), 0, nc * 2, 0x00020000);
        const __amdgpu_buffer_rsrc_t rci = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(sh.col_idx), 0, nc * 4, 0x00020000);
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            bbase[j] = (int)__builtin_amdgcn_raw_buffer_load_b16(rcp, col * 2, 0, 0);
            ocol[j] = __builtin_amdgcn_raw_buffer_load_b32(rci, col * 4, 0, 0);
        }
    } else {
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            const int pos = col < nc ? (int)(sh.col_pos[col] & COL_CELL) - G::TAP0 : 0;
            bbase[j] = pos;
        }
    }
    floatx4 acc[NBA][COH];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int h = 0; h < COH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[j][h][r] = 0.f;

    constexpr int W16 = NSTEP * COH * 64;                        // 16-byte elements of a weight chunk
    constexpr int WPT = (W16 + G::NT - 1) / G::NT;
    typename std::conditional<IL, ItemRegs16<G, ItemRegs<G, bf16_t, BF_CIB>::IPT>, ItemRegs<G, bf16_t, BF_CIB>>::type R;
    intx4w wr[WPT];                    // unconditional buffer loads, see the fp32 kernel
#define APRNET_LOAD_WEIGHTS(q)                                                                     \
    {                                                                                              \
        const __amdgpu_buffer_rsrc_t rw_ = __builtin_amdgcn_make_buffer_rsrc(                      \
            const_cast<uint4*>(wl + (int64_t)(q) * W16), 0, W16 * 16, 0x00020000);                 \
        _Pragma("unroll") for (int k = 0; k < WPT; ++k)                                            \
            wr[k] = __builtin_amdgcn_raw_buffer_load_b128(rw_, (int)(threadIdx.x + k * G::NT) * 16, 0, 0); \
    }
#define APRNET_STORE_WEIGHTS()                                                                     \
    _Pragma("unroll") for (int k = 0; k < WPT; ++k) {                                              \
        const int i = threadIdx.x + k * G::NT;                                                     \
        if (i < W16) reinterpret_cast<intx4w*>(Wl16)[i] = wr[k];                                   \
    }
    if constexpr (IL) {
        fetch_slots16<G, ItemRegs<G, bf16_t, BF_CIB>::IPT, BIG>(sh, nitem, R);
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            bbase[j] = col < nc ? (bbase[j] & (int)COL_CELL) - G::TAP0 : 0;
        }
        load_values16<G, ItemRegs<G, bf16_t, BF_CIB>::IPT, BIG>(a, 0, nitem, tree_items, R);
    } else load_items<G, bf16_t, BF_CIB>(a, 0, nitem, tree_items, sh, R, 0, std::bool_constant<FUSE>{});
    APRNET_LOAD_WEIGHTS(0)
    for (int i = threadIdx.x; i < G::CH_STRIDE; i += G::NT) patch16[i] = make_uint4(0u, 0u, 0u, 0u);     // once per window
    for (int ci0 = 0; ci0 < a.Cin; ci0 += BF_CIB) {
        __syncthreads();
        // items -> patch: one 16-byte cell per item, the eight bfloat16 channels of the chunk
        if constexpr (IL) store_items16<G>(R, nitem, patch16); else store_items_bf16<G>(R, nitem, patch16);
        APRNET_STORE_WEIGHTS()
        __syncthreads();
        if (ci0 + BF_CIB < a.Cin) {
            if constexpr (IL) load_values16<G, ItemRegs<G, bf16_t, BF_CIB>::IPT, BIG>(a, ci0 + BF_CIB, nitem, tree_items, R);
            else load_values<G, bf16_t, BF_CIB>(a, ci0 + BF_CIB, nitem, tree_items, R, 0, std::bool_constant<FUSE>{});
            APRNET_LOAD_WEIGHTS(ci0 / BF_CIB + 1)
        }
#pragma unroll
        for (int st = 0; st < NSTEP; ++st) {
            bf16x8 av[COH];
#pragma unroll
            for (int h = 0; h < COH; ++h) av[h] = __builtin_bit_cast(bf16x8, Wl16[(st * COH + h) * 64 + lane]);
            const int toff = toff_l[st * 4 + (lane >> 4)];       // cell offset of this lane group's tap (4 * step + lane / 16)
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const bf16x8 bv = __builtin_bit_cast(bf16x8, patch16[bbase[j] + toff]);
#pragma unroll
                for (int h = 0; h < COH; ++h) acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[h], bv, acc[j][h], 0, 0, 0);
            }
        }
    }
#undef APRNET_LOAD_WEIGHTS
#undef APRNET_STORE_WEIGHTS
    bf16x8 ha_hi, ha_lo;
    if constexpr (HEAD) {
        ha_hi = __builtin_bit_cast(bf16x8, head_a[lane]);
        ha_lo = __builtin_bit_cast(bf16x8, head_a[64 + lane]);
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
        if constexpr (MODE == 0 && HEAD) {
            // The head as one more matrix product: the lane's channels 4 g .. 4 g + 3 (g = lane / 16) of its column,
            // rounded to bfloat16, are k-slots 8 g .. 8 g + 3 of a B operand (the other four slots are zero), the
            // head's weights the A operand, each fp32 weight as a bfloat16 head plus a bfloat16 remainder (kept to
            // 2^-16, as the stand-alone 1x1x1 kernel of grouped tensors keeps them); sums in fp32.  Output k of
            // column n ends up in register k of lane n.  Every lane takes part (a matrix instruction reads the
            // operand registers of all lanes, also of those whose column lies past the end); only the store is guarded.
            const int g = lane >> 4;
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                v[r] = acc[j][0][r] + bias_l[4 * g + r];
                if (a.relu) v[r] = v[r] < 0.f ? 0.f : v[r];
            }
            const unsigned lo = (unsigned)float_to_bf16(v[0]).bits | ((unsigned)float_to_bf16(v[1]).bits << 16);
            const unsigned hi = (unsigned)float_to_bf16(v[2]).bits | ((unsigned)float_to_bf16(v[3]).bits << 16);
            const bf16x8 bv = __builtin_bit_cast(bf16x8, make_uint4(lo, hi, 0u, 0u));
            floatx4 hacc = {0.f, 0.f, 0.f, 0.f};
            hacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ha_hi, bv, hacc, 0, 0, 0);
            hacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ha_lo, bv, hacc, 0, 0, 0);
            if (g == 0 && col < nc) {
                const int64_t oh = ocol[j];
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    if (k < a.head_C) a.head_y[(int64_t)k * a.head_ld + oh] = float_to_bf16(hacc[k] + head_b4[k]);
            }
            continue;
        }
        if (col >= nc) continue;
        int64_t o;
        if constexpr (IL) o = ocol[j]; else o = sh.col_idx[col];
        if constexpr (MODE == 0) {
            if (IL && a.y_g8) {
                // grouped output: the lane's four channels of a part are half of a 16-byte group
#pragma unroll
                for (int h = 0; h < COH; ++h) {
                    const int c4 = co0 + h * 16 + 4 * (lane >> 4);
                    float v[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        v[r] = acc[j][h][r] + bias_l[h * 16 + 4 * (lane >> 4) + r];
                        if (FUSE && a.relu) v[r] = v[r] < 0.f ? 0.f : v[r];
                    }
                    if (c4 < a.Cout)
                        *reinterpret_cast<uint2*>(a.y + (((int64_t)(c4 >> 3) * a.ldy + o) << 3) + (c4 & 4)) =
                            make_uint2((unsigned)float_to_bf16(v[0]).bits | ((unsigned)float_to_bf16(v[1]).bits << 16),
                                       (unsigned)float_to_bf16(v[2]).bits | ((unsigned)float_to_bf16(v[3]).bits << 16));
                }
                continue;
            }
#pragma unroll
            for (int h = 0; h < COH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int cl = h * 16 + 4 * (lane >> 4) + r;
                    float v = acc[j][h][r] + bias_l[cl];
                    if (FUSE && a.relu) v = v < 0.f ? 0.f : v;
                    if (co0 + cl < a.Cout) a.y[(int64_t)(co0 + cl) * a.ldy + o] = float_to_bf16(v);
                }
        } else {
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

// The windows of the tile come as precomputed lists from the plan.
// Two workgroups per CU (128 registers); the forward pass of layers of at most 16 outputs on regrouped input runs
// three (80 registers, with spills): a third chain of windows per CU hides more of the memory round trips at the
// start of every window than the spills cost (16->16 on the 23 M-particle APR 1.40 -> 1.28 ms; four workgroups at 64
// registers: 2.39 ms; three for 32 outputs: 3.76 against 2.61 ms).
template <class G, int COH, bool FUSE = false, int MODE = 0, bool IL = false, bool BIG = false, bool HEAD = false>
__global__ void __launch_bounds__(G::NT)
__attribute__((amdgpu_waves_per_eu((COH == 1 && MODE == 0 && IL) ? 6 : 4, (COH == 1 && MODE == 0 && IL) ? 6 : 4)))
conv_mfma_bf16_kernel(const ConvArgs<bf16_t> a) {
    constexpr int NBW = 4, NSTEP = bf16_steps<G>();
    static_assert((G::MAXCOL + 15) / 16 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    __shared__ __attribute__((aligned(16))) uint4 patch16[G::CH_STRIDE];
    __shared__ __attribute__((aligned(16))) uint4 Wl16[NSTEP * COH * 64];
    __shared__ float bias_l[16 * COH];

    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level;
    const int co0 = blockIdx.y * 16 * COH;
    const int s_idx = min(a.S_exp - 1, a.Lc - L);
    const int nq = (a.Cin + BF_CIB - 1) / BF_CIB;
    // a.w carries the packed bfloat16 image
    const uint4* __restrict__ wl = reinterpret_cast<const uint4*>(a.w) +
                                   ((int64_t)s_idx * gridDim.y + blockIdx.y) * nq * (NSTEP * COH * 64);
    const int wave = threadIdx.x >> 6;
    const bool tree_items = MODE == 0 && L < a.Lc;       // the output gradient has no tree part

    if (threadIdx.x < 16 * COH)
        bias_l[threadIdx.x] = (MODE == 0 && a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;

    __shared__ int4 hdr[16];                  // headers of sixteen windows: one round trip instead of one per window
    // tap offsets per step and lane group: a table in LDS costs one read per step and saves the registers of a
    // per-lane copy through the whole kernel (the 16-output form no longer spills inside its matrix phase)
    __shared__ int toff_l[NSTEP * 4];
    if (threadIdx.x < NSTEP * 4) toff_l[threadIdx.x] = tap_offset_rt<G>(threadIdx.x);
    __shared__ __attribute__((aligned(16))) uint4 head_a[HEAD ? 128 : 1];
    __shared__ float head_b4[4];
    if constexpr (HEAD) {
        static_assert(COH == 1 && MODE == 0 && IL, "the head follows a forward layer of at most 16 outputs on grouped input");
        const int hs = min(a.head_S - 1, a.Lc - L);
        if (threadIdx.x < 64) {
            // A[m = lane % 16][k = 8 (lane / 16) + i] = head weight of output m and channel 4 (lane / 16) + i for i < 4
            const int m = threadIdx.x & 15, c0 = 4 * (threadIdx.x >> 4);
            unsigned hi16[4], lo16[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float wv = (m < a.head_C && c0 + i < a.Cout) ? a.head_w[((int64_t)hs * a.head_C + m) * a.Cout + c0 + i] : 0.f;
                const bf16_t h = float_to_bf16(wv);
                hi16[i] = h.bits;
                lo16[i] = float_to_bf16(wv - bf16_to_float(h)).bits;
            }
            head_a[threadIdx.x] = make_uint4(hi16[0] | (hi16[1] << 16), hi16[2] | (hi16[3] << 16), 0u, 0u);
            head_a[64 + threadIdx.x] = make_uint4(lo16[0] | (lo16[1] << 16), lo16[2] | (lo16[3] << 16), 0u, 0u);
        }
        if (threadIdx.x < 4) head_b4[threadIdx.x] = (a.head_b && (int)threadIdx.x < a.head_C) ? a.head_b[threadIdx.x] : 0.f;
    }
    const int wb = a.tile_win[blockIdx.x], we = a.tile_win[blockIdx.x + 1];
    for (int w = wb; w < we; ++w) {
        const int win = w - wb;
        if ((win & 15) == 0) {                // every wave is past the previous window's last barrier
            if (threadIdx.x < 16 && w + (int)threadIdx.x < we) hdr[threadIdx.x] = a.win[w + threadIdx.x];
            __syncthreads();
        }
        const int4 hd = hdr[win & 15];
        const int nitem = __builtin_amdgcn_readfirstlane(hd.y), nc = __builtin_amdgcn_readfirstlane(hd.w);
        const unsigned i0 = (unsigned)__builtin_amdgcn_readfirstlane(hd.x), c0 = (unsigned)__builtin_amdgcn_readfirstlane(hd.z);
        const WindowLists gl{a.l_item_idx + i0, a.l_item_pos + i0, a.l_col_idx + c0, a.l_col_pos + c0};
        const int nblk = (nc + 15) >> 4;
        const int first = (wave - (int)blockIdx.x - win) & (G::NWAVE - 1);
        const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;
        switch (__builtin_amdgcn_readfirstlane(nb)) {
            case 0: mfma_bf16_window<G, COH, 0, FUSE, MODE, IL, BIG, HEAD>(a, co0, nc, nitem, tree_items, first, wl, gl, patch16, Wl16, bias_l, toff_l, head_a, head_b4); break;
            case 1: mfma_bf16_window<G, COH, 1, FUSE, MODE, IL, BIG, HEAD>(a, co0, nc, nitem, tree_items, first, wl, gl, patch16, Wl16, bias_l, toff_l, head_a, head_b4); break;
            case 2: mfma_bf16_window<G, COH, 2, FUSE, MODE, IL, BIG, HEAD>(a, co0, nc, nitem, tree_items, first, wl, gl, patch16, Wl16, bias_l, toff_l, head_a, head_b4); break;
            case 3: mfma_bf16_window<G, COH, 3, FUSE, MODE, IL, BIG, HEAD>(a, co0, nc, nitem, tree_items, first, wl, gl, patch16, Wl16, bias_l, toff_l, head_a, head_b4); break;
            default: mfma_bf16_window<G, COH, 4, FUSE, MODE, IL, BIG, HEAD>(a, co0, nc, nitem, tree_items, first, wl, gl, patch16, Wl16, bias_l, toff_l, head_a, head_b4); break;
        }
        __syncthreads();        // the next window rewrites the patch
    }
}

using M333N = ConvGeom<3, 3, 3, 2, 4, 512, 64, 16>;
using M133N = ConvGeom<1, 3, 3, 1, 8, 512, 64, 16>;
using M155N = ConvGeom<1, 5, 5, 1, 8, 512, 64, 16>;
// input gradient of the 3x3x3 stencil: the second patch (box sums) leaves room for two workgroups per CU, so
// each gets 12 waves
using D333N = ConvGeom<3, 3, 3, 2, 4, 768, 64, 16>;

// stencils with a matrix-core kernel (kz*100 + kx*10 + ky); 5x5x5 needs a weight chunk that does not fit LDS
bool conv_mfma_supported(int code) { return code == 333 || code == 133 || code == 155; }
static int conv_taps(int code) { return code == 333 ? 27 : code == 133 ? 9 : 25; }
static int conv_coh(int Cm) { return Cm <= 16 ? 1 : 2; }

// a.tile_win set: forward with the window lists of the plan; otherwise the kernel scans (always for the input gradient)
template <typename T, class G, int MODE>
static int launch16(const ConvArgs<T>& a, int n_tiles, hipStream_t st) {
    const int coh = conv_coh(a.Cout);
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 16 * coh - 1) / (16 * coh)));
    const bool fuse = MODE == 0 && (a.relu || a.x2);
    if (MODE == 0 && a.tile_win && fuse) {
        if (coh == 1) hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 1, 0, true, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 2, 0, true, true>), grid, dim3(G::NT), 0, st, a);
    } else if (MODE == 0 && a.tile_win) {
        if (coh == 1) hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 1, 0, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 2, 0, true>), grid, dim3(G::NT), 0, st, a);
    } else if (fuse) {
        if (coh == 1) hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 1, 0, false, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 2, 0, false, true>), grid, dim3(G::NT), 0, st, a);
    } else if (coh == 1) hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 1, MODE, false>), grid, dim3(G::NT), 0, st, a);
    else hipLaunchKernelGGL((conv_mfma16_kernel<T, G, 2, MODE, false>), grid, dim3(G::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma16_kernel");
    return 0;
}
template <typename T, int MODE>
static int launch16_code(int code, const ConvArgs<T>& a, int n_tiles, hipStream_t st) {
    switch (code) {
        case 333:
            if constexpr (MODE == 1) return launch16<T, D333N, MODE>(a, n_tiles, st);
            else return launch16<T, M333N, MODE>(a, n_tiles, st);
        case 133: return launch16<T, M133N, MODE>(a, n_tiles, st);
        case 155: return launch16<T, M155N, MODE>(a, n_tiles, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "no matrix-core kernel for this stencil");
}

// Forward.  a.w must point at the packed weights (pack_conv_weights).
int launch_conv_mfma(int code, const ConvArgs<float>& a, int n_tiles, hipStream_t st) { return launch16_code<float, 0>(code, a, n_tiles, st); }
// bfloat16 features, fp32 contraction (weights packed by pack_conv_weights)
int launch_conv_mfma(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st) { return launch16_code<bf16_t, 0>(code, a, n_tiles, st); }

// bfloat16 features, bfloat16 contraction (a.w = image of pack_conv_weights_bf16)
template <class G>
static int launch_bf16(const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st, bool dx = false) {
    const int coh = conv_coh(a.Cout);
    dim3 grid((unsigned)n_tiles, (unsigned)((a.Cout + 16 * coh - 1) / (16 * coh)));
    if (dx && a.xi != nullptr) {           // regrouped output gradient
        if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, false, 1, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, false, 1, true>), grid, dim3(G::NT), 0, st, a);
    } else if (dx) {
        if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, false, 1>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, false, 1>), grid, dim3(G::NT), 0, st, a);
    } else if (a.head_w != nullptr) {       // the layer and the 1x1x1 head that follows it, grouped input, at most 16 outputs
        if (a.xi == nullptr || coh != 1) return fail(APRNET_ERR_UNSUPPORTED, "conv_forward: the fused head takes grouped input and at most 16 channels");
        if (a.big) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, true, 0, true, true, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, true, 0, true, false, true>), grid, dim3(G::NT), 0, st, a);
    } else if (a.xi != nullptr && a.big) {   // regrouped input of 2^28 elements and more per group: 64-bit addresses
        if (a.relu) {
            if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, true, 0, true, true>), grid, dim3(G::NT), 0, st, a);
            else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, true, 0, true, true>), grid, dim3(G::NT), 0, st, a);
        } else if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, false, 0, true, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, false, 0, true, true>), grid, dim3(G::NT), 0, st, a);
    } else if (a.xi != nullptr) {          // regrouped input (the second tensor is already part of it)
        if (a.relu) {
            if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, true, 0, true>), grid, dim3(G::NT), 0, st, a);
            else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, true, 0, true>), grid, dim3(G::NT), 0, st, a);
        } else if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, false, 0, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, false, 0, true>), grid, dim3(G::NT), 0, st, a);
    } else if (a.relu || a.x2) {
        if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1, true>), grid, dim3(G::NT), 0, st, a);
        else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2, true>), grid, dim3(G::NT), 0, st, a);
    } else if (coh == 1) hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 1>), grid, dim3(G::NT), 0, st, a);
    else hipLaunchKernelGGL((conv_mfma_bf16_kernel<G, 2>), grid, dim3(G::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_mfma_bf16_kernel");
    return 0;
}
int launch_conv_mfma_bf16(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st) {
    switch (code) {
        case 333: return launch_bf16<M333N>(a, n_tiles, st);
        case 133: return launch_bf16<M133N>(a, n_tiles, st);
        case 155: return launch_bf16<M155N>(a, n_tiles, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "no matrix-core kernel for this stencil");
}
// Input gradient with bfloat16 products: a.x / a.Cin describe the output gradient, a.Cout the layer's input channels,
// a.w the transposed image of pack_conv_weights_bf16, a.tile_win ... the input-gradient lists of the plan.
int launch_conv_dx_mfma_bf16(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st) {
    switch (code) {
        case 333: return launch_bf16<M333N>(a, n_tiles, st, true);
        case 133: return launch_bf16<M133N>(a, n_tiles, st, true);
        case 155: return launch_bf16<M155N>(a, n_tiles, st, true);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "no matrix-core kernel for this stencil");
}
// x (and x2 from channel c_split on) -> out[(C + 7) / 8][count][8]
int interleave8_bf16(const bf16_t* x, int64_t ldx, const bf16_t* x2, int64_t ldx2, int c_split, int C, int64_t count, bf16_t* out,
                     hipStream_t st) {
    if (count <= 0 || C <= 0) return 0;
    dim3 grid((unsigned)std::min<int64_t>((count + 255) / 256, 1 << 20), (unsigned)((C + BF_CIB - 1) / BF_CIB));
    hipLaunchKernelGGL(interleave8_kernel, grid, dim3(256), 0, st, x, ldx, x2, ldx2, c_split, C, count, out);
    APRNET_LAUNCH_CHECK("interleave8_kernel");
    return 0;
}
size_t conv_packed_bf16_bytes(int code, int S_exp, int Cout, int Cin) {
    const int coh = conv_coh(Cout), nstep = (conv_taps(code) + 3) / 4;
    return (size_t)S_exp * ((Cout + 16 * coh - 1) / (16 * coh)) * ((Cin + BF_CIB - 1) / BF_CIB) * nstep * coh * 64 * sizeof(uint4);
}
// Cout / Cin: channels on the M axis of the kernel / contracted channels (transposed: the layer's Cin / Cout)
int pack_conv_weights_bf16(int code, const float* w, int S_exp, int Cout, int Cin, void* packed, hipStream_t st, bool transposed) {
    const size_t n = conv_packed_bf16_bytes(code, S_exp, Cout, Cin) / sizeof(uint4);
    dim3 grid((unsigned)std::min<size_t>((n + 255) / 256, 2048));
    hipLaunchKernelGGL(pack_weights_bf16_kernel, grid, dim3(256), 0, st, w, S_exp, Cout, Cin, conv_taps(code), conv_coh(Cout),
                       transposed ? 1 : 0, (uint4*)packed);
    APRNET_LAUNCH_CHECK("pack_weights_bf16_kernel");
    return 0;
}

// Input gradient: a.x / a.Cin describe the output gradient, a.Cout the input channels, a.w the packed
// transposed weights, a.tiles the row groups within one row of an output (n_tiles of them).
int launch_conv_dx_mfma(int code, const ConvArgs<float>& a, int n_tiles, hipStream_t st) { return launch16_code<float, 1>(code, a, n_tiles, st); }
int launch_conv_dx_mfma(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st) { return launch16_code<bf16_t, 1>(code, a, n_tiles, st); }

// Cm: channels on the M axis of the kernel, Ck: contracted channels (forward: Cout, Cin; transposed: Cin, Cout)
// `transposed`: image for the input gradient (chunks of DX_CIB), otherwise for the forward pass (chunks of FWD_CIB)
size_t conv_packed_floats(int code, int S_exp, int Cm, int Ck, bool transposed) {
    const int coh = conv_coh(Cm), cib = transposed ? DX_CIB : FWD_CIB;
    return (size_t)S_exp * ((Cm + 16 * coh - 1) / (16 * coh)) * ((Ck + cib - 1) / cib) * cib * conv_taps(code) * 16 * coh;
}

int pack_conv_weights(int code, const float* w, int S_exp, int Cm, int Ck, bool transposed, float* packed, hipStream_t st) {
    const size_t n = conv_packed_floats(code, S_exp, Cm, Ck, transposed);
    if (n >= ((size_t)1 << 31)) return fail(APRNET_ERR_UNSUPPORTED, "packed weight image of 2^31 elements or more");
    dim3 grid((unsigned)std::min<size_t>((n + 255) / 256, 2048));
    hipLaunchKernelGGL(pack_weights16_kernel, grid, dim3(256), 0, st, w, S_exp, Cm, Ck, conv_taps(code), transposed ? DX_CIB : FWD_CIB, conv_coh(Cm),
                       transposed ? 1 : 0, packed);
    APRNET_LAUNCH_CHECK("pack_weights16_kernel");
    return 0;
}

}  // namespace aprnet
