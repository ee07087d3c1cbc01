// Stencil convolution forward for layers with very few input channels (1 to 3: the first layer of a network).
//
// Such a layer moves 4 * (Cin + Cout) bytes per particle for 2 * K * Cin * Cout flops: it is bound by memory, and
// by the latency of the gather, not by the contraction.  The general matrix-core kernel (conv_mfma.hip) stages
// chunks of four input channels - three of them zeros here - and runs one window at a time: list header, item
// slots, values, LDS, contraction, stores, every step waiting for the one before.  This kernel is shaped for
// bandwidth instead:
//   * persistent workgroups walk contiguous ranges of the plan's window list, and every global load is issued at
//     least one window before its result is used (header three windows ahead, item slots two, values and output
//     columns one), so the workgroup waits for memory once per window at most and the loads of several windows are
//     in flight per CU.  All loads are unconditional buffer loads (out-of-range lanes read zero) and nothing touches
//     a loaded register before the top of the next iteration: a load under a branch, an operation on its result or a
//     copy of its register would each put a wait for memory into the middle of the window;
//   * the outputs of a window are stored at the start of the next iteration, after its wait, so that no wait
//     includes stores that were issued just before it;
//   * the patch is triple-buffered in LDS (one channel of a window is 6 KB), which leaves one barrier per window;
//   * the contraction runs on v_mfma_f32_16x16x4_f32 with K = (tap, input channel) flattened, so no matrix row
//     multiplies zeros: the four lane groups of an instruction take four consecutive (channel, y-tap) units of one
//     (z, x) row of the stencil - 9 instructions per 16 columns for Cin = 1 instead of 27.  A unit past the end of the
//     row has zero weights and re-reads the row's first unit.
//   * weights of one level stay in LDS (they are re-staged when the window range crosses into another level).
// Same lists, same patch cells, same output layout as the general kernel; every output is written once.
#include "conv_common.hpp"

namespace aprnet {

typedef float floatx4n __attribute__((ext_vector_type(4)));

template <class G, int CIN> struct NarrowShape {
    static constexpr int UNITS = CIN * G::KY;               // (channel, y-tap) units per stencil row
    static constexpr int Q = (UNITS + 3) / 4;               // matrix instructions per stencil row and 16 columns
    static constexpr int ROWS = G::KZ * G::KX;
    static constexpr int STEPS = ROWS * Q;
    static constexpr int IPT = (G::MAXITEM + G::NT - 1) / G::NT;
};

// packed[s][cb][row][q][h][lane]: lane l supplies W[co = (cb * COH + h) * 16 + l % 16][unit 4 q + l / 16 of the row]
__global__ void pack_weights_narrow_kernel(const float* __restrict__ w, int S_exp, int Cout, int Cin, int KY, int ROWS, int Q, int COH,
                                           float* __restrict__ out) {
    const int ncb = (Cout + 16 * COH - 1) / (16 * COH), K = ROWS * KY;
    const unsigned n = (unsigned)S_exp * ncb * ROWS * Q * COH * 64;
    for (unsigned e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        unsigned r = e;
        const int lane = (int)(r % 64u); r /= 64u;
        const int h = (int)(r % (unsigned)COH); r /= (unsigned)COH;
        const int q = (int)(r % (unsigned)Q); r /= (unsigned)Q;
        const int row = (int)(r % (unsigned)ROWS); r /= (unsigned)ROWS;
        const int cb = (int)(r % (unsigned)ncb); r /= (unsigned)ncb;
        const int s = (int)r;
        const int co = (cb * COH + h) * 16 + (lane & 15), u = 4 * q + (lane >> 4);
        float v = 0.f;
        if (u < Cin * KY && co < Cout) {
            const int ci = u / KY, sy = u % KY;
            v = w[(((int64_t)s * Cout + co) * Cin + ci) * K + row * KY + sy];
        }
        out[e] = v;
    }
}

// bfloat16 features, one input channel, 3x3x3 (the first layer of a bfloat16 network): the 27 taps are the K of ONE
// v_mfma_f32_16x16x32_bf16 per 16 columns instead of nine fp32 instructions; weights rounded to bfloat16, as in the
// general bfloat16 kernel.  Slot i (0..7) of lane group g holds tap (row, dy), row = 3 dz + dx:
//     g < 3:  rows 3 g, 3 g + 1 whole (slots 0-2, 3-5) and taps 0, 1 of row 3 g + 2 (slots 6, 7)
//     g = 3:  tap 2 of rows 2, 5, 8 (slots 0, 3, 6); the other slots have zero weights
// so every lane reads three runs of the patch, at cell + base A / B / C (+ 0, 1, 2): the same instructions for all lanes.
__host__ __device__ inline int narrow_bf16_tap(int g, int i) {         // tap index row * 3 + dy of a slot, -1: none
    if (g < 3) return (3 * g + i / 3) * 3 + i % 3;
    return i % 3 == 0 ? (3 * (i / 3) + 2) * 3 + 2 : -1;
}
// packed[s][cb][h][lane]: the lane's 8 bfloat16 of the A operand (output channel (cb * COH + h) * 16 + lane % 16)
__global__ void pack_weights_narrow_bf16_kernel(const float* __restrict__ w, int S_exp, int Cout, int COH, uint4* __restrict__ out) {
    const int ncb = (Cout + 16 * COH - 1) / (16 * COH);
    const unsigned n = (unsigned)S_exp * ncb * COH * 64;
    for (unsigned e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
        unsigned r = e;
        const int lane = (int)(r % 64u); r /= 64u;
        const int h = (int)(r % (unsigned)COH); r /= (unsigned)COH;
        const int cb = (int)(r % (unsigned)ncb); r /= (unsigned)ncb;
        const int s = (int)r;
        const int co = (cb * COH + h) * 16 + (lane & 15), g = lane >> 4;
        unsigned b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int t = narrow_bf16_tap(g, i);
            b[i] = (t >= 0 && co < Cout) ? (unsigned)float_to_bf16(w[((int64_t)s * Cout + co) * 27 + t]).bits : 0u;
        }
        out[e] = make_uint4(b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16));
    }
}

// two workgroups of eight waves per CU (three, at 80 registers with a few spills, ran slower: 2.0 against 1.25 ms)
constexpr int NARROW_WAVES = 4;
struct NarrowArgs {
    int win0;                           // first window of this launch
    int n_win;                          // windows of this launch (stored windows of the plan's lists, finest level first)
    int n_lv;                           // levels with windows
    int lv_first[MAX_LEVELS];           // first window of the k-th such level
    int lv_level[MAX_LEVELS];
};

// TREE: the windows may hold items that come from the tree (any level below the finest one of the call); without
// it the tree loads, a third of a window's load instructions, are not issued at all
// BM: the bfloat16 matrix instruction described above (bfloat16 features, CIN 1, 3x3x3)
typedef __bf16 bf16x8n __attribute__((ext_vector_type(8)));
template <typename T, class G, int CIN, int COH, bool TREE, bool BM = false>
__global__ void __launch_bounds__(G::NT) __attribute__((amdgpu_waves_per_eu(NARROW_WAVES, NARROW_WAVES)))
conv_narrow_kernel(const ConvArgs<T> a, const NarrowArgs na) {
    static_assert(!BM || (std::is_same<T, bf16_t>::value && CIN == 1 && G::KZ == 3 && G::KX == 3 && G::KY == 3), "see narrow_bf16_tap");
    typedef NarrowShape<G, CIN> NS;
    constexpr int IPT = NS::IPT, NBW = ((G::MAXCOL + 15) / 16 + G::NWAVE - 1) / G::NWAVE;
    constexpr int PATCH = CIN * G::CH_STRIDE;
    static_assert((G::MAXCOL + 15) / 16 <= G::NWAVE * NBW, "a window must fit the accumulators of the block");
    __shared__ __attribute__((aligned(16))) float patch[3 * PATCH];
    __shared__ float Wl[BM ? 1 : NS::STEPS * COH * 64];
    __shared__ __attribute__((aligned(16))) uint4 Wl16[BM ? COH * 64 : 1];
    __shared__ float bias_l[16 * COH];

    const int lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int co0 = blockIdx.y * 16 * COH;
    const int wb = na.win0 + (int)((int64_t)na.n_win * blockIdx.x / gridDim.x), we = na.win0 + (int)((int64_t)na.n_win * (blockIdx.x + 1) / gridDim.x);
    if (wb >= we) return;

    if (threadIdx.x < 16 * COH)
        bias_l[threadIdx.x] = (a.bias && co0 + (int)threadIdx.x < a.Cout) ? a.bias[co0 + threadIdx.x] : 0.f;
    for (int i = threadIdx.x; i < 3 * PATCH; i += G::NT) patch[i] = 0.f;

    // per-lane part of the B address: unit u = 4 q + lane / 16 of a stencil row -> channel plane and y-tap
    int loff[NS::Q];
#pragma unroll
    for (int q = 0; q < NS::Q; ++q) {
        int u = 4 * q + (lane >> 4);
        if (u >= NS::UNITS) u = 0;                       // zero weights: any cell the column really reads will do
        loff[q] = (u / G::KY) * G::CH_STRIDE + (u % G::KY) - G::TAP0;
    }

    // BM: the three runs of this lane group, relative to the column's cell
    int runA = 0, runB = 0, runC = 0;
    if constexpr (BM) {
        auto row_off = [](int row) { return ((row / G::KX) * G::RX + (row % G::KX)) * G::RS; };
        const int g = lane >> 4;
        runA = (g < 3 ? row_off(3 * g) : row_off(2) + 2) - G::TAP0;
        runB = (g < 3 ? row_off(3 * g + 1) : row_off(5) + 2) - G::TAP0;
        runC = (g < 3 ? row_off(3 * g + 2) : row_off(8) + 2) - G::TAP0;
    }

    const __amdgpu_buffer_rsrc_t r_hdr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int4*>(a.win), 0, (na.win0 + na.n_win) * 16, 0x00020000);
    __amdgpu_buffer_rsrc_t rx[CIN], rt[CIN];
#pragma unroll
    for (int c = 0; c < CIN; ++c) {
        rx[c] = plane_rsrc<T>(a.x, a.ldx, c, a.Cin, a.x_count);
        rt[c] = plane_rsrc<T>(a.tree_data, a.ldt, c, a.tree_data ? a.Cin : 0, a.t_count);
    }
    typedef int intx4n __attribute__((ext_vector_type(4)));
    // Every load below is an unconditional buffer load whose out-of-range lanes read zero: a load under a branch
    // would be followed by a wait for its result inside the branch, one memory round trip each.
    // header of window w (all lanes read the same 16 bytes; past the end of the range: an empty window)
    auto load_header = [&](int w) -> intx4n {
        return __builtin_amdgcn_raw_buffer_load_b128(r_hdr, w < we ? w * 16 : (int)BUF_OOB, 0, 0);
    };
    // item slots of a window, as loaded: index into the plane (or tree) and patch cell + flags
    struct Slots { int idx[IPT]; int pos[IPT]; };
    auto load_slots = [&](const intx4n hd, Slots& s) {
        const unsigned ib = (unsigned)__builtin_amdgcn_readfirstlane(hd[0]);
        const int nitem = __builtin_amdgcn_readfirstlane(hd[1]);
        const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(a.l_item_idx + ib), 0, nitem * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(a.l_item_pos + ib), 0, nitem * 2, 0x00020000);
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            const int it = threadIdx.x + k * G::NT;
            if (k == 0 || k * G::NT < nitem) {          // wave-uniform: most windows fill one round
                s.idx[k] = __builtin_amdgcn_raw_buffer_load_b32(ri, it * 4, 0, 0);
                s.pos[k] = (int)__builtin_amdgcn_raw_buffer_load_b16(rp, it * 2, 0, 0);
            } else { s.idx[k] = 0; s.pos[k] = 0; }
        }
    };
    // values of the slots' items: a lane past the window's items reads slot zeros and loads element 0 (unused)
    // (from the plane and from the tree with one of the two offsets out of range; the two are combined when the
    // values are used, not here: an operation on a loaded value makes the wave wait for it)
    struct Vals { typename RawLoad<T>::raw x[IPT][CIN], t[TREE ? IPT : 1][CIN]; };
    auto load_vals = [&](const intx4n hd, const Slots& s, Vals& v) {
        const int nitem = __builtin_amdgcn_readfirstlane(hd[1]);
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            if (k > 0 && k * G::NT >= nitem) {              // wave-uniform: a round without items issues no loads
#pragma unroll
                for (int c = 0; c < CIN; ++c) { v.x[k][c] = 0; if constexpr (TREE) v.t[k][c] = 0; }
                continue;
            }
            const unsigned off = (unsigned)s.idx[k] * (unsigned)sizeof(T);
            const bool from_tree = (s.pos[k] & ITEM_TREE) != 0;
            if constexpr (TREE) {
                const unsigned ox = from_tree ? BUF_OOB : off, ot = from_tree ? off : BUF_OOB;
#pragma unroll
                for (int c = 0; c < CIN; ++c) { v.x[k][c] = RawLoad<T>::ld(rx[c], ox); v.t[k][c] = RawLoad<T>::ld(rt[c], ot); }
            } else {
#pragma unroll
                for (int c = 0; c < CIN; ++c) v.x[k][c] = RawLoad<T>::ld(rx[c], off);
            }
        }
    };
    // the columns this wave computes in window w: block j holds columns 16 * (first + NWAVE j) .. + 15
    struct Cols { int idx[NBW]; int pos[NBW]; };
    auto load_cols = [&](const intx4n hd, int w, Cols& c) {
        const unsigned cb = (unsigned)__builtin_amdgcn_readfirstlane(hd[2]);
        const int nc = __builtin_amdgcn_readfirstlane(hd[3]);
        const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(a.l_col_idx + cb), 0, nc * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(a.l_col_pos + cb), 0, nc * 2, 0x00020000);
        const int first = (wave - w) & (G::NWAVE - 1);
#pragma unroll
        for (int j = 0; j < NBW; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            if (j == 0 || ((first + G::NWAVE * j) << 4) < nc) {        // wave-uniform: a block the window does not have issues no loads
                c.idx[j] = __builtin_amdgcn_raw_buffer_load_b32(ri, col * 4, 0, 0);
                c.pos[j] = (int)__builtin_amdgcn_raw_buffer_load_b16(rp, col * 2, 0, 0);
            } else { c.idx[j] = 0; c.pos[j] = 0; }
        }
    };
    auto level_of = [&](int w) -> int {
        int lv = na.lv_level[0];
        for (int k = 1; k < na.n_lv; ++k) if (w >= na.lv_first[k]) lv = na.lv_level[k];
        return lv;
    };
    const int ncb = gridDim.y;
    auto stage_weights = [&](int level) {
        const int s_idx = min(a.S_exp - 1, a.Lc - level);
        if constexpr (BM) {
            const uint4* src16 = reinterpret_cast<const uint4*>(a.w) + ((int64_t)s_idx * ncb + blockIdx.y) * (COH * 64);
            if (threadIdx.x < COH * 64) Wl16[threadIdx.x] = src16[threadIdx.x];
            return;
        }
        const float* src = a.w + ((int64_t)s_idx * ncb + blockIdx.y) * (NS::STEPS * COH * 64);
        for (int i = threadIdx.x; i < NS::STEPS * COH * 64; i += G::NT) Wl[i] = src[i];
    };
    // results of a window: lane l holds column l % 16 of each of its blocks, channels 4 (l / 16) .. + 3 of each
    // 16-channel part.  They are stored at the start of the NEXT iteration, right after its wait for memory, so
    // that no wait of the loop ever includes stores that were issued just before it.
    floatx4n acc[NBW][COH];
    auto store_outputs = [&](const Cols& c, int w, int nc) {
        const int first = (wave - w) & (G::NWAVE - 1);
#pragma unroll
        for (int j = 0; j < NBW; ++j) {
            const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
            if (((first + G::NWAVE * j) << 4) >= nc) break;          // wave-uniform: no such block
            if (col >= nc) continue;
            const int64_t o = c.idx[j];
            if constexpr (std::is_same<T, bf16_t>::value) {
                if (a.y_g8) {          // grouped output [Cout / 8][ldy][8]: the lane's four channels are half of a 16-byte group
#pragma unroll
                    for (int h = 0; h < COH; ++h) {
                        const int c4 = co0 + h * 16 + 4 * (lane >> 4);
                        float v[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            v[r] = acc[j][h][r] + bias_l[h * 16 + 4 * (lane >> 4) + r];
                            if (a.relu) v[r] = v[r] < 0.f ? 0.f : v[r];
                        }
                        if (c4 < a.Cout)
                            *reinterpret_cast<uint2*>(a.y + (((int64_t)(c4 >> 3) * a.ldy + o) << 3) + (c4 & 4)) =
                                make_uint2((unsigned)float_to_bf16(v[0]).bits | ((unsigned)float_to_bf16(v[1]).bits << 16),
                                           (unsigned)float_to_bf16(v[2]).bits | ((unsigned)float_to_bf16(v[3]).bits << 16));
                    }
                    continue;
                }
            }
#pragma unroll
            for (int h = 0; h < COH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int cl = h * 16 + 4 * (lane >> 4) + r;
                    float v = acc[j][h][r] + bias_l[cl];
                    if (a.relu) v = v < 0.f ? 0.f : v;
                    if (co0 + cl < a.Cout) a.y[(int64_t)(co0 + cl) * a.ldy + o] = Num<T>::st(v);
                }
        }
    };

    // ---- prologue: windows wb, wb + 1, wb + 2.  Names ending in N hold what the loop's loads are writing; they are
    // copied to the working names at the top of the next iteration, after its wait (a copy of a register that a load
    // is still writing would wait for that load).
    intx4n h0, h1 = load_header(wb), h2 = load_header(wb + 1), hN = load_header(wb + 2);
    Slots s0, s1, sN;
    Cols cp, c0, cN;
    Vals v0, vN;
    load_slots(h1, s1);
    load_cols(h1, wb, cN);
    load_slots(h2, sN);
    load_vals(h1, s1, vN);
    int cur_level = level_of(wb);
    stage_weights(cur_level);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NBW; ++j) c0.idx[j] = c0.pos[j] = 0;
    int nc_prev = 0, nc = 0;

    typedef const volatile __attribute__((address_space(3))) float lds_float;
    int it = 0;
    for (int w = wb; w < we; ++w, ++it) {
        float* buf = patch + (it % 3) * PATCH;
        // everything that was loaded during the previous iteration: w's header, slots, values and columns become current
        h0 = h1; h1 = h2; h2 = hN; s0 = s1; s1 = sN; cp = c0; c0 = cN; v0 = vN; nc_prev = nc;
        const int nitem = __builtin_amdgcn_readfirstlane(h0[1]);
        nc = __builtin_amdgcn_readfirstlane(h0[3]);
        // 0. outputs of the previous window.  Everything loaded during the previous iteration is waited for here, by
        // hand (vmcnt 0, the other counters untouched): left to the compiler the wait lands at the first use of a
        // loaded value, after these stores, and then includes them (memory operations complete in issue order).
        __builtin_amdgcn_s_waitcnt(0x0F70);
        if (nc_prev > 0) store_outputs(cp, w - 1, nc_prev);
        // 1. the items of this window -> its patch buffer (zeroed two windows ago)
#pragma unroll
        for (int k = 0; k < IPT; ++k) {
            if (k * G::NT >= nitem) break;                  // wave-uniform
            if ((int)threadIdx.x + k * G::NT >= nitem) continue;
            float* cell = buf + ((unsigned)s0.pos[k] & ITEM_CELL);
#pragma unroll
            for (int c = 0; c < CIN; ++c) {
                float v;
                if constexpr (TREE) v = RawLoad<T>::cast(v0.x[k][c] | v0.t[k][c]); else v = RawLoad<T>::cast(v0.x[k][c]);
                cell[c * G::CH_STRIDE] = v;
                if (s0.pos[k] & ITEM_PAIR) cell[c * G::CH_STRIDE + 1] = v;
            }
        }
        // 2. loads of the windows ahead: values of w + 1, columns of w + 1, slots of w + 2, header of w + 3
        load_vals(h1, s1, vN);
        load_cols(h1, w + 1, cN);
        load_slots(h2, sN);
        hN = load_header(w + 3);
        __syncthreads();
        // the buffer of window w + 2 was last read by window w - 1: every wave is past that now
        {
            static_assert(PATCH % 4 == 0, "the patch is cleared with 16-byte stores");
            float4* nz = reinterpret_cast<float4*>(patch + ((it + 2) % 3) * PATCH);
            for (int i = threadIdx.x; i < PATCH / 4; i += G::NT) nz[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        const int level = level_of(w);
        if (level != cur_level) {           // block-uniform
            cur_level = level;
            stage_weights(level);
            __syncthreads();
        }
        // 3. contraction
        const int first = (wave - w) & (G::NWAVE - 1);
        const int nblk = (nc + 15) >> 4;
        const int nb = first < nblk ? (nblk - first + G::NWAVE - 1) / G::NWAVE : 0;
#pragma unroll
        for (int j = 0; j < NBW; ++j)
#pragma unroll
            for (int h = 0; h < COH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][h][r] = 0.f;
        if constexpr (BM) {
            if (nb > 0) {
                lds_float* lp = (lds_float*)buf;
                bf16x8n av[COH];
#pragma unroll
                for (int h = 0; h < COH; ++h) av[h] = __builtin_bit_cast(bf16x8n, Wl16[h * 64 + lane]);
#pragma unroll
                for (int j = 0; j < NBW; ++j) {
                    if (j >= nb) break;                 // wave-uniform
                    const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
                    const int cell = col < nc ? (c0.pos[j] & (int)COL_CELL) : G::TAP0;
                    lds_float* pa = lp + cell + runA; lds_float* pb = lp + cell + runB; lds_float* pc = lp + cell + runC;
                    // the staged values are bfloat16 widened to fp32: the upper halves are the operand
                    const unsigned f0 = __builtin_bit_cast(unsigned, pa[0]), f1 = __builtin_bit_cast(unsigned, pa[1]);
                    const unsigned f2 = __builtin_bit_cast(unsigned, pa[2]), f3 = __builtin_bit_cast(unsigned, pb[0]);
                    const unsigned f4 = __builtin_bit_cast(unsigned, pb[1]), f5 = __builtin_bit_cast(unsigned, pb[2]);
                    const unsigned f6 = __builtin_bit_cast(unsigned, pc[0]), f7 = __builtin_bit_cast(unsigned, pc[1]);
                    const bf16x8n bv = __builtin_bit_cast(bf16x8n, make_uint4(__builtin_amdgcn_perm(f1, f0, 0x07060302u), __builtin_amdgcn_perm(f3, f2, 0x07060302u),
                                                                             __builtin_amdgcn_perm(f5, f4, 0x07060302u), __builtin_amdgcn_perm(f7, f6, 0x07060302u)));
#pragma unroll
                    for (int h = 0; h < COH; ++h) acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[h], bv, acc[j][h], 0, 0, 0);
                }
            }
        } else
        if (nb > 0) {
            lds_float* lp = (lds_float*)buf;
            int bb[NBW][NS::Q];
#pragma unroll
            for (int j = 0; j < NBW; ++j) {
                const int col = ((first + G::NWAVE * j) << 4) + (lane & 15);
                const int cell = col < nc ? (c0.pos[j] & (int)COL_CELL) : G::TAP0;
#pragma unroll
                for (int q = 0; q < NS::Q; ++q) bb[j][q] = cell + loff[q];
            }
            const float* ap = Wl + lane;
#pragma unroll
            for (int row = 0; row < NS::ROWS; ++row) {
                const int roff = ((row / G::KX) * G::RX + (row % G::KX)) * G::RS;
#pragma unroll
                for (int q = 0; q < NS::Q; ++q) {
                    float av[COH];
#pragma unroll
                    for (int h = 0; h < COH; ++h) av[h] = ap[((row * NS::Q + q) * COH + h) * 64];
#pragma unroll
                    for (int j = 0; j < NBW; ++j) {
                        if (j >= nb) break;             // wave-uniform
                        const float bv = lp[bb[j][q] + roff];
#pragma unroll
                        for (int h = 0; h < COH; ++h) acc[j][h] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[h], bv, acc[j][h], 0, 0, 0);
                    }
                }
            }
        }
    }
    if (nc > 0) store_outputs(c0, we - 1, nc);
}

using N333 = ConvGeom<3, 3, 3, 2, 4, 512, 64, 16>;
using N133 = ConvGeom<1, 3, 3, 1, 8, 512, 64, 16>;
using N155 = ConvGeom<1, 5, 5, 1, 8, 512, 64, 16>;

constexpr int NARROW_MAX_CIN = 3;
bool conv_narrow_supported(int code, int Cin) { return (code == 333 || code == 133 || code == 155) && Cin >= 1 && Cin <= NARROW_MAX_CIN; }

template <class G> static void narrow_dims(int Cin, int* rows, int* q) {
    *rows = G::KZ * G::KX; *q = (Cin * G::KY + 3) / 4;
}
static int narrow_coh(int Cout) { return Cout <= 16 ? 1 : 2; }

// bfloat16 features on the bfloat16 matrix instruction (see narrow_bf16_tap)
int bf16_math();
bool conv_narrow_bf16_math(int code, int Cin) { return bf16_math() && code == 333 && Cin == 1; }
size_t conv_narrow_packed_floats(int code, int S_exp, int Cout, int Cin, bool bf16m) {
    if (bf16m) { const int coh = Cout <= 16 ? 1 : 2; return (size_t)S_exp * ((Cout + 16 * coh - 1) / (16 * coh)) * coh * 64 * 4; }
    int rows, q;
    if (code == 333) narrow_dims<N333>(Cin, &rows, &q); else if (code == 133) narrow_dims<N133>(Cin, &rows, &q); else narrow_dims<N155>(Cin, &rows, &q);
    const int coh = narrow_coh(Cout);
    return (size_t)S_exp * ((Cout + 16 * coh - 1) / (16 * coh)) * rows * q * coh * 64;
}

int pack_conv_weights_narrow(int code, const float* w, int S_exp, int Cout, int Cin, float* packed, hipStream_t st, bool bf16m) {
    if (bf16m) {
        const size_t n16 = conv_narrow_packed_floats(code, S_exp, Cout, Cin, true) / 4;
        hipLaunchKernelGGL(pack_weights_narrow_bf16_kernel, dim3((unsigned)std::min<size_t>((n16 + 255) / 256, 1024)), dim3(256), 0, st, w, S_exp,
                           Cout, Cout <= 16 ? 1 : 2, reinterpret_cast<uint4*>(packed));
        APRNET_LAUNCH_CHECK("pack_weights_narrow_bf16_kernel");
        return 0;
    }
    int rows, q;
    if (code == 333) narrow_dims<N333>(Cin, &rows, &q); else if (code == 133) narrow_dims<N133>(Cin, &rows, &q); else narrow_dims<N155>(Cin, &rows, &q);
    const size_t n = conv_narrow_packed_floats(code, S_exp, Cout, Cin, false);
    const int ky = code % 10;
    hipLaunchKernelGGL(pack_weights_narrow_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 1024)), dim3(256), 0, st, w, S_exp, Cout, Cin,
                       ky, rows, q, narrow_coh(Cout), packed);
    APRNET_LAUNCH_CHECK("pack_weights_narrow_kernel");
    return 0;
}

template <typename T, class G, int CIN>
static int launch_narrow_cin(const ConvArgs<T>& a, const NarrowArgs& na, hipStream_t st) {
    const int coh = narrow_coh(a.Cout);
    // two persistent workgroups per CU; short lists get one workgroup per window
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    // the windows of the call's finest level hold no tree items (they come first in the list): their launch skips the tree loads
    const int n_fine = (na.n_lv > 0 && na.lv_level[0] == a.Lc) ? (na.n_lv > 1 ? na.lv_first[1] : na.n_win) : 0;
    for (int part = 0; part < 2; ++part) {
        NarrowArgs nb = na;
        nb.win0 = part == 0 ? 0 : n_fine;
        nb.n_win = part == 0 ? n_fine : na.n_win - n_fine;
        if (nb.n_win <= 0) continue;
        dim3 grid((unsigned)std::max(1, std::min(nb.n_win, 2 * cus)), (unsigned)((a.Cout + 16 * coh - 1) / (16 * coh)));
        if constexpr (std::is_same<T, bf16_t>::value && CIN == 1 && G::KZ == 3) {
            if (conv_narrow_bf16_math(333, 1)) {
                if (part == 0) {
                    if (coh == 1) hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 1, false, true>), grid, dim3(G::NT), 0, st, a, nb);
                    else hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 2, false, true>), grid, dim3(G::NT), 0, st, a, nb);
                } else {
                    if (coh == 1) hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 1, true, true>), grid, dim3(G::NT), 0, st, a, nb);
                    else hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 2, true, true>), grid, dim3(G::NT), 0, st, a, nb);
                }
                APRNET_LAUNCH_CHECK("conv_narrow_kernel");
                continue;
            }
        }
        if (part == 0) {
            if (coh == 1) hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 1, false>), grid, dim3(G::NT), 0, st, a, nb);
            else hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 2, false>), grid, dim3(G::NT), 0, st, a, nb);
        } else {
            if (coh == 1) hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 1, true>), grid, dim3(G::NT), 0, st, a, nb);
            else hipLaunchKernelGGL((conv_narrow_kernel<T, G, CIN, 2, true>), grid, dim3(G::NT), 0, st, a, nb);
        }
        APRNET_LAUNCH_CHECK("conv_narrow_kernel");
    }
    return 0;
}
template <typename T, class G>
static int launch_narrow_g(const ConvArgs<T>& a, const NarrowArgs& na, hipStream_t st) {
    switch (a.Cin) {
        case 1: return launch_narrow_cin<T, G, 1>(a, na, st);
        case 2: return launch_narrow_cin<T, G, 2>(a, na, st);
        case 3: return launch_narrow_cin<T, G, 3>(a, na, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "narrow convolution kernel: 1 to 3 input channels");
}
template <typename T>
static int launch_narrow(int code, const ConvArgs<T>& a, const WinLists& wl, hipStream_t st) {
    if (wl.n_win <= 0) return 0;
    NarrowArgs na{};
    na.n_win = wl.n_win; na.n_lv = wl.n_lv;
    for (int k = 0; k < wl.n_lv; ++k) { na.lv_first[k] = wl.lv_first[k]; na.lv_level[k] = wl.lv_level[k]; }
    switch (code) {
        case 333: return launch_narrow_g<T, N333>(a, na, st);
        case 133: return launch_narrow_g<T, N133>(a, na, st);
        case 155: return launch_narrow_g<T, N155>(a, na, st);
    }
    return fail(APRNET_ERR_UNSUPPORTED, "narrow convolution kernel: no such stencil");
}
// a.w: image of pack_conv_weights_narrow; a.l_* / a.win: the plan's window lists (wl)
int launch_conv_narrow(int code, const ConvArgs<float>& a, const WinLists& wl, hipStream_t st) { return launch_narrow<float>(code, a, wl, st); }
int launch_conv_narrow(int code, const ConvArgs<bf16_t>& a, const WinLists& wl, hipStream_t st) { return launch_narrow<bf16_t>(code, a, wl, st); }

}  // namespace aprnet
