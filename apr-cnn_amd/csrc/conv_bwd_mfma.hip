// Stencil convolution backward on the matrix cores (fp32 MFMA), gfx950: gradient of the weights.
// (The gradient of the input is the forward kernel run on the output gradient with the transposed,
// flipped stencil, conv_mfma.hip.)
//
//   dW[s][co][ci][t] = sum over output positions (columns) of  gY[co][col] * patch[ci][pos(col) + off(t)]
//
// is a GEMM with M = 32 output channels, N = taps (27 of the 32 columns of the tile are used) and the
// columns of the window as the contracted axis, one 32x32 accumulator per input channel:
//
//     v_mfma_f32_32x32x2_f32:  D[co][t] += A[co][k] * B[k][t],   k = two columns of the window
//       A: lane l supplies gY[co = l%32] of column k = l/32      (LDS image gyl, laid out so that the
//                                                                  read is linear in the lane index)
//       B: lane l supplies patch[ci][pos(column k = l/32) + off(t = l%32)]
//
// A block owns 16 input channels (four staged chunks of 4) and 32 output channels.  Wave w takes input
// channel w%4 of every chunk and half of the columns (w/4), so it holds four accumulators, and keeps them
// in registers while the (persistent) block walks over many tiles of one stencil index (one launch per
// stencil index); they are added to the result with one atomic per element at the end.  The patch rows are 67 words
// apart so that the 27 tap offsets of a B read fall into 27 different LDS banks.
#include "conv_common.hpp"

namespace aprnet {

typedef float floatx16 __attribute__((ext_vector_type(16)));
int bf16_math();       // conv.hip: bfloat16 features multiply on the bfloat16 matrix instructions (default) or in fp32

// row strides that put the tap offsets of one B read into different banks: 67 for 3-wide, 69 for 5-wide rows
using W333M = ConvGeom<3, 3, 3, 2, 4, 512, 67>;
using W133M = ConvGeom<1, 3, 3, 1, 8, 512, 67>;
using W155M = ConvGeom<1, 5, 5, 1, 8, 512, 69>;
constexpr int DW_CIB = 4;          // input channels per staged chunk
constexpr int DW_NCH = 4;          // chunks per block
constexpr int DW_GB = 256;         // columns of gY staged at a time
constexpr int DW_KB = 8;          // MFMAs issued back to back between operand phases (16 would spill registers)
constexpr int DW_GLD = 33;         // words per column of gyl (32 output channels + 1 against bank conflicts)

// Lists of the plan carry patch cells for rows of 64 words; this kernel's rows are RS words apart.
template <class G> __device__ __forceinline__ unsigned restride(unsigned pos) {
    return (pos & ~ITEM_CELL) | (((pos & ITEM_CELL) >> 6) * G::RS + (pos & 63u));
}

// Output gradient of one group of up to DW_GB columns -> LDS (through `put`), and the patch cell of every column of the
// group -> cpl.  Wave w takes output channels co0 + w, co0 + w + NWAVE, ... (NCO of them) of 64 columns per batch.
// The loads come in two rounds for the whole group -- column indices and cells of all batches (unconditional buffer
// loads, lanes past the group read zero), then the gradient values, those of batch b + 1 issued before the LDS stores
// of batch b -- instead of five dependent round trips per batch: a load under `c < ng`, or under `idx >= 0`, followed
// by its use makes the compiler wait for memory on the spot.
template <typename T, class G, int NCO, bool LISTS, class Lists, class Put>
__device__ __forceinline__ void stage_gy_group(const ConvArgs<T>& a, const Lists& sh, int g0, int ng, int co0, int co_end, int wave,
                                               int lane, int* __restrict__ cpl, Put put) {
    constexpr int NBM = DW_GB / 64;
    const int nbatch = (ng + 63) >> 6;
    int idx[NBM], pos[NBM];
    if constexpr (LISTS) {
        const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(sh.col_idx + g0), 0, ng * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(sh.col_pos + g0), 0, ng * 2, 0x00020000);
#pragma unroll
        for (int b = 0; b < NBM; ++b) {
            idx[b] = __builtin_amdgcn_raw_buffer_load_b32(ri, (b * 64 + lane) * 4, 0, 0);
            pos[b] = (int)__builtin_amdgcn_raw_buffer_load_b16(rp, (b * 64 + lane) * 2, 0, 0);
        }
    } else {
#pragma unroll
        for (int b = 0; b < NBM; ++b) {
            const int c = b * 64 + lane;
            idx[b] = c < ng ? sh.col_idx[g0 + c] : 0;
            pos[b] = c < ng ? (int)sh.col_pos[g0 + c] : 0;
        }
    }
    if (wave == 0) {        // patch cell of every column of the group, as a word offset
#pragma unroll
        for (int b = 0; b < NBM; ++b) {
            if (b >= nbatch) break;
            const int c = b * 64 + lane;
            cpl[c] = c < ng ? (LISTS ? (int)restride<G>((unsigned)pos[b]) : pos[b]) : G::TAP0;
        }
    }
    T cur[NCO], nxt[NCO];
    auto load = [&](int b, T (&v)[NCO]) {
#pragma unroll
        for (int k = 0; k < NCO; ++k) {
            const int co = co0 + wave + k * G::NWAVE;
            // (a lane past the group reads element 0 of the plane; its value is replaced by zero below)
            v[k] = a.gy[(int64_t)min(co, co_end - 1) * a.ldy + idx[b]];
        }
    };
    load(0, cur);
#pragma unroll
    for (int b = 0; b < NBM; ++b) {
        if (b >= nbatch) break;
        if (b + 1 < nbatch) load(b + 1 < NBM ? b + 1 : b, nxt);
        const int c = b * 64 + lane;
#pragma unroll
        for (int k = 0; k < NCO; ++k) {
            const int co = wave + k * G::NWAVE;
            put(b, c, co, cur[k], c < ng && co0 + co < co_end);
        }
#pragma unroll
        for (int k = 0; k < NCO; ++k) cur[k] = nxt[k];
    }
}

// One window: its output gradient goes to gyl in groups of DW_GB columns; per group the four channel chunks of
// the block are staged one after the other (the loads of the next chunk are issued before the matrix phase of
// the current one) and contracted with the group's columns.
template <typename T, class G, int CIB, int NCH, bool LISTS, class Lists>
__device__ __forceinline__ void dw_window(const ConvArgs<T>& a, const Lists& sh, int nc, int nitem, bool tree_items,
                                          int cig0, int co0, int bl, int kh, int hi, int wave, int lane,
                                          float* __restrict__ patch, float* __restrict__ gyl, int* __restrict__ cpl,
                                          const float* ap, floatx16 (&acc)[NCH]) {
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    ItemRegs<G, T, CIB> R;
    fetch_slots<G, T, CIB>(sh, nitem, R);
    if constexpr (LISTS) {
#pragma unroll
        for (int k = 0; k < ItemRegs<G, T, CIB>::IPT; ++k)
            if (R.pos[k] != 0xffffu) R.pos[k] = (unsigned short)restride<G>(R.pos[k]);
    }
    load_values<G, T, CIB>(a, cig0, nitem, tree_items, R);
    for (int g0 = 0; g0 < nc; g0 += DW_GB) {
        const int ng = min(DW_GB, nc - g0), nbatch = (ng + 63) >> 6;
        // output gradient of this group of columns -> gyl; a wave reads 64 columns of one channel
        stage_gy_group<T, G, 32 / G::NWAVE, LISTS>(a, sh, g0, ng, co0, a.Cout, wave, lane, cpl,
            [&](int b, int, int co, T v, bool valid) {
                const int slot = b * 64 + 2 * (lane & 31) + (lane >> 5);
                gyl[slot * DW_GLD + co] = valid ? Num<T>::ld(v) : 0.f;
            });
#pragma unroll
        for (int q = 0; q < NCH; ++q) {
            __syncthreads();        // previous chunk's reads of the patch are done / gyl is written
            store_items<G, T, CIB>(R, nitem, patch);
            __syncthreads();
            if (q + 1 < NCH) load_values<G, T, CIB>(a, cig0 + (q + 1) * CIB, nitem, tree_items, R);
            else if (g0 + DW_GB < nc) load_values<G, T, CIB>(a, cig0, nitem, tree_items, R);     // next group starts over
#pragma unroll 1
            for (int b = 0; b < nbatch; ++b) {
                const float* apb = ap + (b * 64 + 32 * kh) * DW_GLD;
                // Three separate phases, kept apart by scheduling barriers: operand addresses (one LDS read of the
                // column's cell and one vector add each), then the operand reads, then DW_KB MFMAs back to back.  A
                // vector instruction between two fp32 MFMAs costs a pipeline switch each time.
                const int* cp = cpl + b * 64 + 32 * hi + 16 * kh;      // lanes of the upper half take column k + 32
#pragma unroll
                for (int h = 0; h < 16; h += DW_KB) {
                    int addr[DW_KB];
#pragma unroll
                    for (int k = 0; k < DW_KB; ++k) addr[k] = bl + cp[h + k];
                    __builtin_amdgcn_sched_barrier(0);
                    float av[DW_KB], bv[DW_KB];
#pragma unroll
                    for (int k = 0; k < DW_KB; ++k) { av[k] = apb[2 * (h + k) * DW_GLD]; bv[k] = patch[addr[k]]; }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int k = 0; k < DW_KB; ++k) acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[k], bv[k], acc[q], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        __syncthreads();            // gyl is rewritten by the next group, the patch by the next window
    }
}

// ---------------------------------------------------------------------------------------------------------
// Layers of at most 16 output channels (the finest stages of the networks): the 32-row instruction above would
// multiply 16 rows of zeros.  Here D is 16 output channels x 16 taps on v_mfma_f32_16x16x4_f32, two tap tiles per
// input channel (taps 0-15 and 16-31), four columns per instruction:
//     A: lane l supplies gY[co = l%16] of column l/16 of the four            (gyl16[column][co], 17 words per column:
//                                                                              conflict-free writes by column, reads
//                                                                              with a few two-way conflicts)
//     B: lane l supplies patch[ci][cell(column l/16) + off(t = l%16 + 16 * tile)]
// Twice the columns per matrix-pipe cycle of the 32x32x2 form for such layers; same staging, same work split
// (wave w: input channel w%4 of each chunk, half w/4 of every 64 columns).
typedef float floatx4d __attribute__((ext_vector_type(4)));
constexpr int DW_GLD16 = 17;

template <typename T, class G, int CIB, int NCH, bool LISTS, class Lists>
__device__ __forceinline__ void dw_window16(const ConvArgs<T>& a, const Lists& sh, int nc, int nitem, bool tree_items,
                                            int cig0, const int (&bl)[2], int kh, int wave, int lane,
                                            float* __restrict__ patch, float* __restrict__ gyl, int* __restrict__ cpl,
                                            floatx4d (&acc)[NCH][2]) {
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0.f;     // once per window
    ItemRegs<G, T, CIB> R;
    fetch_slots<G, T, CIB>(sh, nitem, R);
    if constexpr (LISTS) {
#pragma unroll
        for (int k = 0; k < ItemRegs<G, T, CIB>::IPT; ++k)
            if (R.pos[k] != 0xffffu) R.pos[k] = (unsigned short)restride<G>(R.pos[k]);
    }
    load_values<G, T, CIB>(a, cig0, nitem, tree_items, R);
    const int q4 = lane >> 4;                                   // which of the four columns of an instruction
    const float* ap = gyl + q4 * DW_GLD16 + (lane & 15);
    for (int g0 = 0; g0 < nc; g0 += DW_GB) {
        const int ng = min(DW_GB, nc - g0), nbatch = (ng + 63) >> 6;
        stage_gy_group<T, G, 16 / G::NWAVE, LISTS>(a, sh, g0, ng, 0, a.Cout, wave, lane, cpl,
            [&](int, int c, int co, T v, bool valid) { gyl[c * DW_GLD16 + co] = valid ? Num<T>::ld(v) : 0.f; });
#pragma unroll
        for (int q = 0; q < NCH; ++q) {
            __syncthreads();        // previous chunk's reads of the patch are done / gyl is written
            store_items<G, T, CIB>(R, nitem, patch);
            __syncthreads();
            if (q + 1 < NCH) load_values<G, T, CIB>(a, cig0 + (q + 1) * CIB, nitem, tree_items, R);
            else if (g0 + DW_GB < nc) load_values<G, T, CIB>(a, cig0, nitem, tree_items, R);     // next group starts over
#pragma unroll 1
            for (int b = 0; b < nbatch; ++b) {
                const int c0 = b * 64 + 32 * kh;                 // this wave's 32 columns of the batch
                if (c0 >= ng) break;                             // wave-uniform: nothing but padding left
                const int* cp = cpl + c0 + q4;
                const float* apb = ap + c0 * DW_GLD16;
                int cell[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) cell[k] = cp[4 * k];
                __builtin_amdgcn_sched_barrier(0);
                float av[8], b0[8], b1[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) { av[k] = apb[4 * k * DW_GLD16]; b0[k] = patch[bl[0] + cell[k]]; b1[k] = patch[bl[1] + cell[k]]; }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    acc[q][0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[k], b0[k], acc[q][0], 0, 0, 0);
                    acc[q][1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[k], b1[k], acc[q][1], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        __syncthreads();            // gyl is rewritten by the next group, the patch by the next window
    }
}

template <typename T, class G, int CIB, int NCH, bool LISTS>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(4, 4)))
conv_dw16_mfma_kernel(const ConvArgs<T> a, const int s_idx) {
    static_assert(G::NWAVE == 8 && CIB == 4, "wave w owns input channel w%4 and column half w/4");
    __shared__ float patch[CIB * G::CH_STRIDE];
    __shared__ float gyl[DW_GB * DW_GLD16];
    __shared__ int cpl[DW_GB];

    const int cig0 = blockIdx.y * (CIB * NCH);
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cil = wave & 3, kh = wave >> 2;
    int bl[2];
#pragma unroll
    for (int tile = 0; tile < 2; ++tile) {
        const int t = (lane & 15) + 16 * tile;
        const int tt = t < G::K ? t : 0;
        const int toff = ((tt / (G::KX * G::KY)) * G::RX + (tt / G::KY) % G::KX) * G::RS + (tt % G::KY);
        bl[tile] = cil * G::CH_STRIDE - G::TAP0 + toff;       // B operand: + cell of the column
    }
    floatx4d acc[NCH][2];
#pragma unroll
    for (int q = 0; q < NCH; ++q)
#pragma unroll
        for (int tile = 0; tile < 2; ++tile)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[q][tile][r] = 0.f;

    for (int ti = blockIdx.x; ti < a.n_tiles; ti += gridDim.x) {
        const ConvTile tile = a.tiles[ti];
        const int L = tile.level;
        const bool tree_items = L < a.Lc;
        if constexpr (LISTS) {
            const int wb = a.tile_win[ti], we = a.tile_win[ti + 1];
            for (int w = wb; w < we; ++w) {
                const int4 hd = a.win[w];
                const int nitem = __builtin_amdgcn_readfirstlane(hd.y), nc = __builtin_amdgcn_readfirstlane(hd.w);
                const WindowLists gl{a.l_item_idx + (unsigned)hd.x, a.l_item_pos + (unsigned)hd.x, a.l_col_idx + (unsigned)hd.z,
                                     a.l_col_pos + (unsigned)hd.z};
                dw_window16<T, G, CIB, NCH, true>(a, gl, nc, nitem, tree_items, cig0, bl, kh, wave, lane, patch, gyl, cpl, acc);
            }
        } else {
            __shared__ ConvShared<G> sh;
            const int yn = a.apr.y_num[L];
            const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
            __syncthreads();
            open_segments<G, T>(a, L, tile.z0, tile.x0, sh);
            __syncthreads();
            for (int y0 = 0; y0 < yn; y0 += G::TY) {
                scan_window<G, T>(a, L, y0, out_tree, sh);
                __syncthreads();
                const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
                if (nc > 0) dw_window16<T, G, CIB, NCH, false>(a, sh, nc, nitem, tree_items, cig0, bl, kh, wave, lane, patch, gyl, cpl, acc);
                __syncthreads();
                close_window<G>(sh);
                __syncthreads();
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NCH; ++q) {
        const int ci = cig0 + q * CIB + cil;
#pragma unroll
        for (int tile = 0; tile < 2; ++tile)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int co = 4 * (lane >> 4) + r, t = (lane & 15) + 16 * tile;
                if (t < G::K && ci < a.Cin && co < a.Cout) {
                    const int64_t e = ((int64_t)co * a.Cin + ci) * G::K + t;
                    if (a.gw_part) a.gw_part[(int64_t)(2 * blockIdx.x + kh) * a.gw_part_ld + e] = acc[q][tile][r];
                    else if (acc[q][tile][r] != 0.f) unsafeAtomicAdd(a.gw + (int64_t)s_idx * a.Cout * a.Cin * G::K + e, acc[q][tile][r]);
                }
            }
    }
}

// ---------------------------------------------------------------------------------------------------------
// bfloat16 features and output gradient: the same contraction on v_mfma_f32_32x32x16_bf16 (16 columns per
// instruction, fp32 accumulation).  Both operands are bfloat16 values as loaded, so the products are the exact
// ones the fp32 kernel forms; only the order of the fp32 sums differs.
//     A: lane l supplies gY[co = l%32] of columns 8*(l/32) .. +7 of a group of 16: one 16-byte read from
//        gyl16[co][column] (rows DW_LDG16 apart)
//     B: lane l supplies patch16[ci][cell(column) + off(t = l%32)] of the same 8 columns: 8 two-byte reads
// An instruction does the work of eight of the fp32 ones, so the loop is bound by its LDS reads.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr int DW_LDG16 = DW_GB + 8;            // 16-byte aligned rows, 4 banks apart

template <class G, int CIB, int NCH, bool LISTS, class Lists>
__device__ __forceinline__ void dw_window_bf16(const ConvArgs<bf16_t>& a, const Lists& sh, int nc, int nitem, bool tree_items,
                                               int cig0, int co0, int bl, int kh, int hi, int wave, int lane,
                                               unsigned short* __restrict__ patch, unsigned short* __restrict__ gyl,
                                               int* __restrict__ cpl, floatx16 (&acc)[NCH]) {
    for (int i = threadIdx.x; i < CIB * G::CH_STRIDE / 2; i += G::NT) reinterpret_cast<unsigned*>(patch)[i] = 0u;   // once per window
    ItemRegs<G, bf16_t, CIB> R;
    fetch_slots<G, bf16_t, CIB>(sh, nitem, R);
    if constexpr (LISTS) {
#pragma unroll
        for (int k = 0; k < ItemRegs<G, bf16_t, CIB>::IPT; ++k)
            if (R.pos[k] != 0xffffu) R.pos[k] = (unsigned short)restride<G>(R.pos[k]);
    }
    load_values<G, bf16_t, CIB>(a, cig0, nitem, tree_items, R);
    for (int g0 = 0; g0 < nc; g0 += DW_GB) {
        const int ng = min(DW_GB, nc - g0), nbatch = (ng + 63) >> 6;
        stage_gy_group<bf16_t, G, 32 / G::NWAVE, LISTS>(a, sh, g0, ng, co0, a.Cout, wave, lane, cpl,
            [&](int, int c, int co, bf16_t v, bool valid) { gyl[co * DW_LDG16 + c] = valid ? v.bits : (unsigned short)0; });
#pragma unroll
        for (int q = 0; q < NCH; ++q) {
            __syncthreads();        // previous chunk's reads of the patch are done / gyl is written
#pragma unroll
            for (int k = 0; k < ItemRegs<G, bf16_t, CIB>::IPT; ++k) {
                if (k * G::NT >= nitem) break;       // wave-uniform
                if (R.pos[k] == 0xffffu) continue;
                unsigned short* cell = patch + (R.pos[k] & ITEM_CELL);
#pragma unroll
                for (int c = 0; c < CIB; ++c) {
                    const unsigned short v = (unsigned short)R.v[k][c];
                    cell[c * G::CH_STRIDE] = v;
                    if (R.pos[k] & ITEM_PAIR) cell[c * G::CH_STRIDE + 1] = v;
                }
            }
            __syncthreads();
            if (q + 1 < NCH) load_values<G, bf16_t, CIB>(a, cig0 + (q + 1) * CIB, nitem, tree_items, R);
            else if (g0 + DW_GB < nc) load_values<G, bf16_t, CIB>(a, cig0, nitem, tree_items, R);     // next group starts over
#pragma unroll 1
            for (int b = 0; b < nbatch; ++b) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int c0 = b * 64 + 32 * kh + 16 * s;           // first of this instruction's 16 columns
                    if (c0 >= ng) break;                                // wave-uniform: nothing but padding left
                    const int4 ca = *reinterpret_cast<const int4*>(cpl + c0 + 8 * hi);
                    const int4 cb = *reinterpret_cast<const int4*>(cpl + c0 + 8 * hi + 4);
                    const int cell[8] = {ca.x, ca.y, ca.z, ca.w, cb.x, cb.y, cb.z, cb.w};
                    unsigned w[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        w[j] = (unsigned)patch[bl + cell[2 * j]] | ((unsigned)patch[bl + cell[2 * j + 1]] << 16);
                    const uint4 av = *reinterpret_cast<const uint4*>(gyl + (lane & 31) * DW_LDG16 + c0 + 8 * hi);
                    const uint4 bv = make_uint4(w[0], w[1], w[2], w[3]);
                    acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, bv),
                                                                     acc[q], 0, 0, 0);
                }
            }
        }
        __syncthreads();            // gyl is rewritten by the next group, the patch by the next window
    }
}

template <class G, int CIB, int NCH, bool LISTS>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(4, 4)))
conv_dw_bf16_kernel(const ConvArgs<bf16_t> a, const int s_idx) {
    static_assert(G::NWAVE == 8 && CIB == 4, "wave w owns input channel w%4 and column half w/4");
    static_assert(G::CH_STRIDE % 2 == 0 && DW_LDG16 % 8 == 0, "dword fill of the patch, 16-byte rows of gyl");
    __shared__ __attribute__((aligned(16))) unsigned short patch[CIB * G::CH_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short gyl[32 * DW_LDG16];
    __shared__ __attribute__((aligned(16))) int cpl[DW_GB];

    const int cig0 = blockIdx.y * (CIB * NCH), co0 = blockIdx.z * 32;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cil = wave & 3, kh = wave >> 2;
    const int t = lane & 31, hi = lane >> 5;
    const int tt = t < G::K ? t : 0;
    const int toff = ((tt / (G::KX * G::KY)) * G::RX + (tt / G::KY) % G::KX) * G::RS + (tt % G::KY);
    const int bl = cil * G::CH_STRIDE - G::TAP0 + toff;       // B operand: + cell of the column

    floatx16 acc[NCH];
#pragma unroll
    for (int q = 0; q < NCH; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[q][r] = 0.f;

    for (int ti = blockIdx.x; ti < a.n_tiles; ti += gridDim.x) {
        const ConvTile tile = a.tiles[ti];
        const int L = tile.level;
        const bool tree_items = L < a.Lc;
        if constexpr (LISTS) {
            const int wb = a.tile_win[ti], we = a.tile_win[ti + 1];
            for (int w = wb; w < we; ++w) {
                const int4 hd = a.win[w];
                const int nitem = __builtin_amdgcn_readfirstlane(hd.y), nc = __builtin_amdgcn_readfirstlane(hd.w);
                const WindowLists gl{a.l_item_idx + (unsigned)hd.x, a.l_item_pos + (unsigned)hd.x, a.l_col_idx + (unsigned)hd.z,
                                     a.l_col_pos + (unsigned)hd.z};
                dw_window_bf16<G, CIB, NCH, true>(a, gl, nc, nitem, tree_items, cig0, co0, bl, kh, hi, wave, lane, patch, gyl, cpl, acc);
            }
        } else {
            __shared__ ConvShared<G> sh;
            const int yn = a.apr.y_num[L];
            const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
            __syncthreads();
            open_segments<G, bf16_t>(a, L, tile.z0, tile.x0, sh);
            __syncthreads();
            for (int y0 = 0; y0 < yn; y0 += G::TY) {
                scan_window<G, bf16_t>(a, L, y0, out_tree, sh);
                __syncthreads();
                const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
                if (nc > 0) dw_window_bf16<G, CIB, NCH, false>(a, sh, nc, nitem, tree_items, cig0, co0, bl, kh, hi, wave, lane, patch, gyl, cpl, acc);
                __syncthreads();
                close_window<G>(sh);
                __syncthreads();
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NCH; ++q) {
        const int ci = cig0 + q * CIB + cil;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int co = co0 + 8 * (r >> 2) + 4 * hi + (r & 3);
            if (t < G::K && ci < a.Cin && co < a.Cout) {
                const int64_t e = ((int64_t)co * a.Cin + ci) * G::K + t;
                if (a.gw_part) a.gw_part[(int64_t)(2 * blockIdx.x + kh) * a.gw_part_ld + e] = acc[q][r];
                else if (acc[q][r] != 0.f) unsafeAtomicAdd(a.gw + (int64_t)s_idx * a.Cout * a.Cin * G::K + e, acc[q][r]);
            }
        }
    }
}

// T: storage type of the features and of the output gradient (float, or bfloat16 widened to fp32 on load).
// LISTS: the windows come from the plan's lists; otherwise the block scans the access arrays.
template <typename T, class G, int CIB, int NCH, bool LISTS>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(4, 4)))
conv_dw_mfma_kernel(const ConvArgs<T> a, const int s_idx) {
    static_assert(G::NWAVE == 8 && CIB == 4, "wave w owns input channel w%4 and column half w/4");
    __shared__ float patch[CIB * G::CH_STRIDE];
    __shared__ float gyl[DW_GB * DW_GLD];
    __shared__ int cpl[DW_GB];

    const int cig0 = blockIdx.y * (CIB * NCH), co0 = blockIdx.z * 32;
    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cil = wave & 3, kh = wave >> 2;
    const int t = lane & 31, hi = lane >> 5;
    const int tt = t < G::K ? t : 0;
    const int toff = ((tt / (G::KX * G::KY)) * G::RX + (tt / G::KY) % G::KX) * G::RS + (tt % G::KY);
    const int bl = cil * G::CH_STRIDE - G::TAP0 + toff;       // B operand: + cell of the column
    const float* ap = gyl + lane + hi;                        // A operand: + (64 * batch + 2 * kk) * DW_GLD

    floatx16 acc[NCH];
#pragma unroll
    for (int q = 0; q < NCH; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[q][r] = 0.f;

    for (int ti = blockIdx.x; ti < a.n_tiles; ti += gridDim.x) {
        const ConvTile tile = a.tiles[ti];
        const int L = tile.level;
        const bool tree_items = L < a.Lc;
        if constexpr (LISTS) {
            const int wb = a.tile_win[ti], we = a.tile_win[ti + 1];
            for (int w = wb; w < we; ++w) {
                const int4 hd = a.win[w];
                const int nitem = __builtin_amdgcn_readfirstlane(hd.y), nc = __builtin_amdgcn_readfirstlane(hd.w);
                const WindowLists gl{a.l_item_idx + (unsigned)hd.x, a.l_item_pos + (unsigned)hd.x, a.l_col_idx + (unsigned)hd.z,
                                     a.l_col_pos + (unsigned)hd.z};
                dw_window<T, G, CIB, NCH, true>(a, gl, nc, nitem, tree_items, cig0, co0, bl, kh, hi, wave, lane, patch, gyl, cpl, ap, acc);
            }
        } else {
            __shared__ ConvShared<G> sh;
            const int yn = a.apr.y_num[L];
            const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
            __syncthreads();
            open_segments<G, T>(a, L, tile.z0, tile.x0, sh);
            __syncthreads();
            for (int y0 = 0; y0 < yn; y0 += G::TY) {
                scan_window<G, T>(a, L, y0, out_tree, sh);
                __syncthreads();
                const int nc = __builtin_amdgcn_readfirstlane(sh.ncol), nitem = __builtin_amdgcn_readfirstlane(sh.nitem);
                if (nc > 0) dw_window<T, G, CIB, NCH, false>(a, sh, nc, nitem, tree_items, cig0, co0, bl, kh, hi, wave, lane, patch, gyl, cpl, ap, acc);
                __syncthreads();
                close_window<G>(sh);
                __syncthreads();
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NCH; ++q) {
        const int ci = cig0 + q * CIB + cil;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int co = co0 + 8 * (r >> 2) + 4 * hi + (r & 3);
            if (t < G::K && ci < a.Cin && co < a.Cout) {
                const int64_t e = ((int64_t)co * a.Cin + ci) * G::K + t;
                if (a.gw_part) a.gw_part[(int64_t)(2 * blockIdx.x + kh) * a.gw_part_ld + e] = acc[q][r];
                else if (acc[q][r] != 0.f) unsafeAtomicAdd(a.gw + (int64_t)s_idx * a.Cout * a.Cin * G::K + e, acc[q][r]);
            }
        }
    }
}

// gw[e] += sum of part[slot][e] over the slots, in slot order: one thread per element, coalesced over e.
__global__ void dw_reduce_kernel(const float* __restrict__ part, int64_t ld, int slots, int64_t n, float* __restrict__ gw) {
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        int k = 0;
        for (; k + 3 < slots; k += 4) {
            s0 += part[(int64_t)k * ld + e]; s1 += part[(int64_t)(k + 1) * ld + e];
            s2 += part[(int64_t)(k + 2) * ld + e]; s3 += part[(int64_t)(k + 3) * ld + e];
        }
        for (; k < slots; ++k) s0 += part[(int64_t)k * ld + e];
        gw[e] += (s0 + s1) + (s2 + s3);
    }
}

// Workgroups of one weight-gradient launch when its partial sums go to a buffer: at most 512, fewer for very wide
// layers so that the buffer (two slots per workgroup) stays within 512 MiB.
int conv_dw_partial_blocks(int code, int Cout, int Cin) {
    const int64_t e = (int64_t)Cout * Cin * (code == 333 ? 27 : code == 133 ? 9 : 25);
    const int64_t cap = ((int64_t)512 << 20) / (8 * e);
    return (int)std::max<int64_t>(16, std::min<int64_t>(512, cap));
}
size_t conv_dw_partial_bytes(int code, int Cout, int Cin) {
    const int64_t e = (int64_t)Cout * Cin * (code == 333 ? 27 : code == 133 ? 9 : 25);
    return (size_t)(2 * conv_dw_partial_blocks(code, Cout, Cin)) * e * sizeof(float);
}

// Weight gradient; a.gw is accumulated into (the caller zeroes it).
// One launch per stencil index: level Lc - s for s < S_exp - 1, every coarser level for the last one
// (adjacent in the tile list, which is sorted finest level first).
template <typename T, class G>
static int launch_dw(const ConvArgs<T>& a0, const TileList& tl, int level_min, hipStream_t st) {
    for (int s = 0; s < a0.S_exp; ++s) {
        const int l_hi = a0.Lc - s, l_lo = (s == a0.S_exp - 1) ? level_min : l_hi;
        if (l_hi < level_min) break;
        int n = 0;
        for (int l = l_lo; l <= l_hi; ++l) n += tl.level_count[l];
        if (n == 0) continue;
        ConvArgs<T> a = a0;
        a.tiles = tl.d_tiles + tl.level_begin[l_hi]; a.n_tiles = n;
        if (a.tile_win) a.tile_win += tl.level_begin[l_hi];
        // a narrow input (the first layer of a network) fits one chunk: no staging and products of empty chunks
        const int nch = a.Cin <= DW_CIB ? 1 : DW_NCH;
        const int gmax = a.gw_part ? a.gw_part_blocks : 512;
        dim3 grid((unsigned)std::min(n, gmax), (unsigned)((a.Cin + DW_CIB * nch - 1) / (DW_CIB * nch)), (unsigned)((a.Cout + 31) / 32));
        const int64_t n_el = (int64_t)a.Cout * a.Cin * G::K;
        // the partial sums of this launch, added up in slot order (every slot of the grid is written in full)
        auto reduce = [&]() -> int {
            if (!a.gw_part) return 0;
            hipLaunchKernelGGL(dw_reduce_kernel, dim3((unsigned)std::min<int64_t>((n_el + 255) / 256, 2048)), dim3(256), 0, st,
                               (const float*)a.gw_part, a.gw_part_ld, 2 * (int)grid.x, n_el, (float*)a.gw + (int64_t)s * n_el);
            APRNET_LAUNCH_CHECK("dw_reduce_kernel");
            return 0;
        };
        if constexpr (std::is_same<T, bf16_t>::value) {
            if (bf16_math()) {      // bfloat16 matrix instructions; the fp32 ones below when those are asked for
                if (nch == 1) {
                    if (a.tile_win) hipLaunchKernelGGL((conv_dw_bf16_kernel<G, DW_CIB, 1, true>), grid, dim3(G::NT), 0, st, a, s);
                    else hipLaunchKernelGGL((conv_dw_bf16_kernel<G, DW_CIB, 1, false>), grid, dim3(G::NT), 0, st, a, s);
                } else if (a.tile_win) hipLaunchKernelGGL((conv_dw_bf16_kernel<G, DW_CIB, DW_NCH, true>), grid, dim3(G::NT), 0, st, a, s);
                else hipLaunchKernelGGL((conv_dw_bf16_kernel<G, DW_CIB, DW_NCH, false>), grid, dim3(G::NT), 0, st, a, s);
                APRNET_LAUNCH_CHECK("conv_dw_bf16_kernel");
                if (int rc = reduce()) return rc;
                continue;
            }
        }
        if (a.Cout <= 16) {         // 16-row form
            if (nch == 1) {
                if (a.tile_win) hipLaunchKernelGGL((conv_dw16_mfma_kernel<T, G, DW_CIB, 1, true>), grid, dim3(G::NT), 0, st, a, s);
                else hipLaunchKernelGGL((conv_dw16_mfma_kernel<T, G, DW_CIB, 1, false>), grid, dim3(G::NT), 0, st, a, s);
            } else if (a.tile_win) hipLaunchKernelGGL((conv_dw16_mfma_kernel<T, G, DW_CIB, DW_NCH, true>), grid, dim3(G::NT), 0, st, a, s);
            else hipLaunchKernelGGL((conv_dw16_mfma_kernel<T, G, DW_CIB, DW_NCH, false>), grid, dim3(G::NT), 0, st, a, s);
            APRNET_LAUNCH_CHECK("conv_dw16_mfma_kernel");
            if (int rc = reduce()) return rc;
            continue;
        }
        if (nch == 1) {
            if (a.tile_win) hipLaunchKernelGGL((conv_dw_mfma_kernel<T, G, DW_CIB, 1, true>), grid, dim3(G::NT), 0, st, a, s);
            else hipLaunchKernelGGL((conv_dw_mfma_kernel<T, G, DW_CIB, 1, false>), grid, dim3(G::NT), 0, st, a, s);
        } else if (a.tile_win) hipLaunchKernelGGL((conv_dw_mfma_kernel<T, G, DW_CIB, DW_NCH, true>), grid, dim3(G::NT), 0, st, a, s);
        else hipLaunchKernelGGL((conv_dw_mfma_kernel<T, G, DW_CIB, DW_NCH, false>), grid, dim3(G::NT), 0, st, a, s);
        APRNET_LAUNCH_CHECK("conv_dw_mfma_kernel");
        if (int rc = reduce()) return rc;
    }
    return 0;
}

template <typename T>
static int launch_dw_code(int code, const ConvArgs<T>& a, const TileList& tl, int level_min, hipStream_t st) {
    switch (code) {
        case 333: return launch_dw<T, W333M>(a, tl, level_min, st);
        case 133: return launch_dw<T, W133M>(a, tl, level_min, st);
        case 155: return launch_dw<T, W155M>(a, tl, level_min, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "no matrix-core kernel for this stencil");
}
int launch_conv_dw_mfma(int code, const ConvArgs<float>& a, const TileList& tl, int level_min, hipStream_t st) {
    return launch_dw_code<float>(code, a, tl, level_min, st);
}
int launch_conv_dw_mfma(int code, const ConvArgs<bf16_t>& a, const TileList& tl, int level_min, hipStream_t st) {
    return launch_dw_code<bf16_t>(code, a, tl, level_min, st);
}

}  // namespace aprnet
