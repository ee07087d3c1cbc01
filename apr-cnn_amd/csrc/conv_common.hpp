// Shared pieces of the stencil convolution kernels: tile geometry, the three-source row gather
// into an LDS patch, and the output-column list.
//
// Work decomposition.  One workgroup owns a row group of one level: TZ x TX sparse rows
// (z0..z0+TZ-1, x0..x0+TX-1) and walks along y in windows of TY output cells.  For each window it
// stages the isotropic neighbourhood of the group, (TZ+KZ-1) x (TX+KX-1) rows of WY = TY+KY-1 = 64
// cells, into LDS.  A staged row is the union of three sorted sparse sources
// (helpers.hpp:358-420):
//     0  particles of the same level            row (L,   z,   x)
//     1  particles one level coarser, each      row (L-1, z/2, x/2)   -> cells 2y, 2y+1
//     2  tree nodes of the same level           tree row (L, z, x)    -> value from the feature
//        vector (L == Lc, "downsampled particles") or from the mean-filled tree (L < Lc)
// and zero elsewhere (outside the image, or not covered).
//
// Each (row, source) pair is a "segment" with a cursor into y_vec that only moves forward.  A window
// holds at most 64 cells, so one 64-lane load of y_vec at the cursor sees every particle of the
// segment that can fall into the window; wave ballots over "y < bound" give the in-window count and
// the cursor advance without any search.
#pragma once
#include "common.hpp"

#include <type_traits>

namespace aprnet {

template <typename T>
struct ConvArgs {
    AccessDev apr, tree;
    const ConvTile* tiles;
    const T* x; int64_t ldx; int Cin;
    // forward only: channels c_split .. Cin - 1 of the input come from a second tensor (x2 null: all from x), and
    // the result can be clamped at zero after the bias
    const T* x2; int64_t ldx2; int c_split; int relu;
    const typename Num<T>::acc* w; int S_exp; int Cout;     // [S_exp][Cout][Cin][K]; fp32 for bfloat16 features
    const typename Num<T>::acc* bias;                       // [Cout] or null
    T* y; int64_t ldy;
    const T* tree_data; int64_t ldt;
    int Lc; int64_t tree_off;                  // tree_offset(Lc)
    int64_t x_count, t_count;                  // valid elements per channel plane of x / tree_data
    // bfloat16 forward only: the input (both tensors) and the tree values regrouped as [Cin / 8][count][8], one
    // 16-byte load per item and group of 8 channels (null: the kernel reads the channel planes)
    const T* xi; const T* ti;
    int64_t xi_ld, ti_ld;                      // particles between two groups of xi / ti
    const T* xi2; int64_t xi2_ld;              // grouped second input: groups from c_split / 8 on (null: all groups in xi)
    int y_g8;                                  // bfloat16 forward: the output is grouped too, [Cout / 8][ldy][8]
    int big;                                   // bfloat16 forward on grouped input: 64-bit addresses (2^28 elements and more per group)
    // bfloat16 forward on grouped input, at most 16 outputs: a 1x1x1 convolution of the result (after bias and clamp,
    // rounded to bfloat16 as a stored result would be) follows inside the kernel and only its output is stored, as
    // planes head_y [head_C][head_ld]; head_w [head_S][head_C][Cout] and head_b [head_C] (or null) in fp32; head_C <= 4.
    // y is not written.  (null head_w: no head)
    const float* head_w; const float* head_b; T* head_y; int64_t head_ld; int head_C, head_S;
    // backward only
    // gradients are accumulated in the computation type (fp32 for bfloat16 features)
    const T* gy; typename Num<T>::acc* gx; int64_t ldgx; typename Num<T>::acc* gtree; int64_t ldgt;
    typename Num<T>::acc* gw; int n_tiles;
    // Weight gradient without atomics: every persistent workgroup writes the sums of its tiles to two slots (one per
    // half of the columns) of gw_part [2 * gw_part_blocks][gw_part_ld], which a second kernel adds up in slot order and
    // adds to gw, so the result does not depend on scheduling (null: atomic additions to gw).
    typename Num<T>::acc* gw_part; int64_t gw_part_ld; int gw_part_blocks;
    // input-gradient scan: leave out the coarser particles that stick out of a far face of the level (some of the
    // cells they would cover do not exist); a separate kernel adds their gradient (faces.hip)
    int dx_skip_faces;
    // window lists built once per APR and kept in the plan (kernels that do not scan)
    const int* tile_win;                       // [n_tiles + 1] first stored window of every tile
    const int4* win;                           // per stored window: {first item, items, first column, columns}; the two
                                               // "first" fields are unsigned 32-bit offsets
    const int* l_item_idx; const unsigned short* l_item_pos;
    const int* l_col_idx; const unsigned short* l_col_pos;
};

// The lists of one window in global memory; same member names as ConvShared, so the staging code takes either.
struct WindowLists {
    const int* item_idx; const unsigned short* item_pos;
    const int* col_idx; const unsigned short* col_pos;
};

template <int KZ_, int KX_, int KY_, int TZ_, int TX_, int NT_, int RS_ = 64, int PAD_ = 32>
struct ConvGeom {
    static constexpr int KZ = KZ_, KX = KX_, KY = KY_, TZ = TZ_, TX = TX_, NT = NT_;
    static constexpr int RS = RS_;                // words between two staged rows of one channel (>= WY)
    static constexpr int K = KZ * KX * KY;
    static constexpr int HZ = (KZ - 1) / 2, HX = (KX - 1) / 2, HY = (KY - 1) / 2;
    static constexpr int RZ = TZ + KZ - 1, RX = TX + KX - 1;
    static constexpr int WY = 64;                 // staged cells per row = one wavefront
    static constexpr int TY = WY - (KY - 1);      // output cells per window
    static constexpr int NROW = RZ * RX;
    static constexpr int NSEG = NROW * 3;
    static constexpr int NWAVE = NT / 64;
    static constexpr int SPW = (NSEG + NWAVE - 1) / NWAVE;     // segments per wave
    static constexpr int MAXCOL = TZ * TX * TY;
    static constexpr int MAXITEM = NROW * WY;                  // every staged cell is filled by at most one item
    static constexpr int ITER = (MAXCOL + NT - 1) / NT;        // output columns per thread
    // patch elements per channel; the extra PAD words put the channels that one MFMA operand read touches
    // (lanes l and l+32 read the same cell of adjacent channels, PAD 32; four lane groups of 16 read four
    // channels, PAD 16) on different parts of the 64 LDS banks
    static constexpr int CH_STRIDE = (NROW * RS + 63) / 64 * 64 + PAD_;
    static constexpr int TAP0 = (HZ * RX + HX) * RS + HY;      // centre -> first tap
};

__device__ __forceinline__ int lane_id() { return __lane_id(); }

// Per-block bookkeeping kept in LDS.
//
// A window is described by two lists that phase A (scan_window) builds once and every channel chunk
// reuses:
//   items   every particle / tree node that falls into the staged window: where its value comes from
//           (feature index, or tree index with ITEM_TREE) and which patch cell(s) it fills;
//   columns the output positions: feature index and centre cell.
// Staging a chunk is then a flat loop over the items with all lanes busy and every global load
// independent of the others (one memory round trip per chunk), instead of one partially filled
// 64-lane load per segment.
template <class G>
struct ConvShared {
    int seg_cur[G::NSEG];            // cursor: first particle of the segment that can fall into the next window
    int seg_end[G::NSEG];
    int col_idx[G::MAXCOL];
    unsigned short col_pos[G::MAXCOL];
    int item_idx[G::MAXITEM];
    unsigned short item_pos[G::MAXITEM];   // bits 0-11 cell inside one channel of the patch, ITEM_PAIR, ITEM_TREE
    int ncol, nitem;
    int nbox;                        // input gradient: pooled columns (COL_BOX) of the window
};

constexpr unsigned ITEM_CELL = 0x0fffu;   // first patch cell the value goes to
constexpr unsigned ITEM_PAIR = 0x1000u;   // coarser particle: the value also fills the next cell
constexpr unsigned ITEM_TREE = 0x2000u;   // value is read from the mean-filled tree, not from the features

// Opens the 3 * NROW segments of a tile.
template <class G, typename T>
__device__ __forceinline__ void open_segments(const ConvArgs<T>& a, int L, int z0, int x0, ConvShared<G>& sh) {
    const int zn = a.apr.z_num[L], xn = a.apr.x_num[L];
    const bool has_parent = L > a.apr.level_min;
    const bool has_tree = L < a.apr.level_max;
    for (int s = threadIdx.x; s < G::NSEG; s += G::NT) {
        const int r = s / 3, src = s - 3 * r;
        const int rz = r / G::RX, rx = r - rz * G::RX;
        const int z = z0 - G::HZ + rz, x = x0 - G::HX + rx;
        int b = 0, e = 0;
        if (z >= 0 && z < zn && x >= 0 && x < xn) {
            if (src == 0) {
                const uint64_t row = a.apr.row(L, z, x);
                b = (int)a.apr.xz_end[row - 1]; e = (int)a.apr.xz_end[row];
            } else if (src == 1) {
                if (has_parent) {
                    const uint64_t row = a.apr.row(L - 1, z >> 1, x >> 1);
                    b = (int)a.apr.xz_end[row - 1]; e = (int)a.apr.xz_end[row];
                }
            } else if (has_tree) {
                const uint64_t row = a.tree.row(L, z, x);
                b = (int)a.tree.xz_end[row - 1]; e = (int)a.tree.xz_end[row];
            }
        }
        sh.seg_cur[s] = b; sh.seg_end[s] = e;
    }
    if (threadIdx.x == 0) { sh.ncol = 0; sh.nitem = 0; sh.nbox = 0; }
}

// Segments are scanned in groups of GRP: the y_vec loads of a group are issued before the first LDS
// write of the group, so a group costs one memory round trip instead of one per segment.
template <class G> struct SegGroup { static constexpr int GRP = G::SPW < 6 ? G::SPW : 6; };

// Phase A of a window.  Every wave loads y_vec at the cursor of its segments (64 lanes = every particle
// that can fall into the 64-cell window).  Ballots over "y < bound" give the number of in-window
// particles (the first n lanes, y ascends) and the cursor of the next window, which is committed at
// once.  In-window particles are appended to the item list; those of the centre rows (plus tree nodes
// when they are downsampled particles) whose y lies in the output range also to the column list.
// Not inlined on purpose: inlined, the per-segment constants of the unrolled loops are hoisted out of the
// window loop and stay live through the contraction, which costs ~80 registers per lane.
struct ScanArgs {
    const uint16_t* apr_y;
    const uint16_t* tree_y;
    int tree_off, yn, y0;
    bool tree_from_x, out_tree;
    int z0, x0, zn, xn;             // tile origin and level extent (input-gradient scan only)
    bool pool;                      // input-gradient scan: one pooled column per coarser particle (COL_BOX)
    bool skip_faces;                // input-gradient scan: no columns for coarser particles with cells outside the level
};

template <class G>
__device__ __attribute__((noinline)) void scan_window_impl(const ScanArgs a, ConvShared<G>& sh);

template <class G, typename T>
__device__ __forceinline__ void scan_window(const ConvArgs<T>& a, int L, int y0, bool out_tree, ConvShared<G>& sh) {
    ScanArgs s;
    s.apr_y = a.apr.y; s.tree_y = a.tree.y; s.tree_off = (int)a.tree_off; s.yn = a.apr.y_num[L]; s.y0 = y0;
    s.tree_from_x = (L == a.Lc); s.out_tree = out_tree;
    scan_window_impl<G>(s, sh);
}

template <class G>
__device__ __attribute__((noinline)) void scan_window_impl(const ScanArgs a, ConvShared<G>& sh) {
    const int y0 = a.y0, yn = a.yn;
    const bool tree_from_x = a.tree_from_x, out_tree = a.out_tree;
    constexpr int GRP = SegGroup<G>::GRP;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int lo = y0 - G::HY, hi = y0 + G::TY + G::HY, lo_next = y0 + G::TY - G::HY;
    for (int k0 = 0; k0 < G::SPW; k0 += GRP) {
        int yy[GRP], cur[GRP];
#pragma unroll
        for (int g = 0; g < GRP; ++g) {
            const int s = wave + (k0 + g) * G::NWAVE;
            yy[g] = INT_MAX; cur[g] = 0;
            if (s < G::NSEG) {
                cur[g] = sh.seg_cur[s];
                const int i = cur[g] + lane;
                if (i < sh.seg_end[s]) yy[g] = (s % 3 == 2) ? (int)a.tree_y[i] : (int)a.apr_y[i];
            }
        }
#pragma unroll
        for (int g = 0; g < GRP; ++g) {
            const int s = wave + (k0 + g) * G::NWAVE;
            if (s >= G::NSEG) break;
            const bool valid = yy[g] != INT_MAX;
            if (__ballot(valid) == 0) continue;                         // wave-uniform: segment is exhausted
            const int r = s / 3, src = s - 3 * r;
            const bool in = valid && (src == 1 ? yy[g] <= ((hi - 1) >> 1) : yy[g] < hi);
            const bool below = valid && (src == 1 ? yy[g] < (lo_next >> 1) : yy[g] < lo_next);
            const unsigned long long m_in = __ballot(in);
            const int n_adv = __popcll(__ballot(below));
            if (lane == 0 && n_adv) sh.seg_cur[s] = cur[g] + n_adv;
            if (m_in == 0) continue;                                    // wave-uniform
            const int i = cur[g] + lane;
            int ibase = 0;
            if (lane == 0) ibase = atomicAdd(&sh.nitem, __popcll(m_in));
            ibase = __shfl(ibase, 0);
            if (in) {      // in-window lanes are lanes 0 .. n_in-1
                unsigned pos;
                if (src != 1) {
                    pos = (unsigned)(r * G::RS + (yy[g] - lo));
                    if (src == 2 && !tree_from_x) pos |= ITEM_TREE;
                } else {
                    const int ya = 2 * yy[g], yb = ya + 1;
                    const bool wa = ya >= lo, wb = yb < hi && yb < yn;
                    pos = (unsigned)(r * G::RS + ((wa ? ya : yb) - lo));
                    if (wa && wb) pos |= ITEM_PAIR;
                }
                sh.item_idx[ibase + lane] = i + ((src == 2 && tree_from_x) ? (int)a.tree_off : 0);
                sh.item_pos[ibase + lane] = (unsigned short)pos;
            }
            const int rz = r / G::RX, rx = r - rz * G::RX;
            const bool centre = rz >= G::HZ && rz < G::HZ + G::TZ && rx >= G::HX && rx < G::HX + G::TX;
            const bool out_seg = centre && (src == 0 || (src == 2 && out_tree));
            const bool outl = out_seg && in && yy[g] >= y0 && yy[g] < y0 + G::TY;
            const unsigned long long m = __ballot(outl);
            if (m) {
                int base = 0;
                if (lane == 0) base = atomicAdd(&sh.ncol, __popcll(m));
                base = __shfl(base, 0);
                if (outl) {
                    const int rank = __popcll(m & ((1ull << lane) - 1ull));
                    sh.col_idx[base + rank] = i + (src == 2 ? (int)a.tree_off : 0);
                    sh.col_pos[base + rank] = (unsigned short)(r * G::RS + (yy[g] - lo));
                }
            }
        }
    }
}

// Phase A of a window for the gradient with respect to the input, in gather form.  The gradient of the
// staged patch is  gV[ci][cell] = sum_{co,t} w[co][ci][t] * gY[co][cell - off(t)],  a convolution of the
// output gradient laid out by position (zero where the level has no output) with the flipped stencil.
//   items    the output positions of the window including the halo rows: same-level particles, and tree
//            nodes where they are downsampled particles;  idx addresses the output gradient
//   columns  every cell of the centre rows that some source covers, with the place its gradient goes to:
//            the same-level particle, the coarser particle, the downsampled particle, or (COL_TREE) the node
//            of the tree-gradient buffer.  A coarser particle collects the gradients of the BOXZ x 2 x 2 cells
//            it covers inside the tile; by linearity that sum is the stencil applied to the box-summed output
//            gradient, so it takes ONE column (COL_BOX, at its first cell) that reads a second patch holding
//            those box sums.  Only at the far faces of the image, where some of the cells do not exist, it
//            takes one column per cell.
constexpr unsigned COL_CELL = 0x0fffu;
constexpr unsigned COL_BOX = 0x4000u;
constexpr unsigned COL_TREE = 0x8000u;

template <class G>
__device__ __attribute__((noinline)) void scan_window_dx_impl(const ScanArgs a, ConvShared<G>& sh) {
    const int y0 = a.y0, yn = a.yn;
    const bool tree_from_x = a.tree_from_x, out_tree = a.out_tree;
    constexpr int GRP = SegGroup<G>::GRP;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int lo = y0 - G::HY, hi = y0 + G::TY + G::HY, lo_next = y0 + G::TY - G::HY;
    const unsigned long long below_me = (1ull << lane) - 1ull;
    for (int k0 = 0; k0 < G::SPW; k0 += GRP) {
        int yy[GRP], cur[GRP];
#pragma unroll
        for (int g = 0; g < GRP; ++g) {
            const int s = wave + (k0 + g) * G::NWAVE;
            yy[g] = INT_MAX; cur[g] = 0;
            if (s < G::NSEG) {
                cur[g] = sh.seg_cur[s];
                const int i = cur[g] + lane;
                if (i < sh.seg_end[s]) yy[g] = (s % 3 == 2) ? (int)a.tree_y[i] : (int)a.apr_y[i];
            }
        }
#pragma unroll
        for (int g = 0; g < GRP; ++g) {
            const int s = wave + (k0 + g) * G::NWAVE;
            if (s >= G::NSEG) break;
            const bool valid = yy[g] != INT_MAX;
            if (__ballot(valid) == 0) continue;                         // wave-uniform: segment is exhausted
            const int r = s / 3, src = s - 3 * r;
            const bool in = valid && (src == 1 ? yy[g] <= ((hi - 1) >> 1) : yy[g] < hi);
            const bool below = valid && (src == 1 ? yy[g] < (lo_next >> 1) : yy[g] < lo_next);
            const unsigned long long m_in = __ballot(in);
            const int n_adv = __popcll(__ballot(below));
            if (lane == 0 && n_adv) sh.seg_cur[s] = cur[g] + n_adv;
            if (m_in == 0) continue;                                    // wave-uniform
            const int i = cur[g] + lane;
            if (src == 0 || (src == 2 && out_tree)) {
                int ibase = 0;
                if (lane == 0) ibase = atomicAdd(&sh.nitem, __popcll(m_in));
                ibase = __shfl(ibase, 0);
                if (in) {
                    sh.item_idx[ibase + lane] = i + (src == 2 ? (int)a.tree_off : 0);
                    sh.item_pos[ibase + lane] = (unsigned short)(r * G::RS + (yy[g] - lo));
                }
            }
            const int rz = r / G::RX, rx = r - rz * G::RX;
            const bool centre = rz >= G::HZ && rz < G::HZ + G::TZ && rx >= G::HX && rx < G::HX + G::TX;
            if (!centre) continue;
            if (src != 1) {
                const bool outl = in && yy[g] >= y0 && yy[g] < y0 + G::TY;
                const unsigned long long m = __ballot(outl);
                if (m) {
                    int base = 0;
                    if (lane == 0) base = atomicAdd(&sh.ncol, __popcll(m));
                    base = __shfl(base, 0);
                    if (outl) {
                        const int rank = __popcll(m & below_me);
                        const bool to_tree = src == 2 && !tree_from_x;
                        sh.col_idx[base + rank] = i + ((src == 2 && tree_from_x) ? (int)a.tree_off : 0);
                        sh.col_pos[base + rank] = (unsigned short)((r * G::RS + (yy[g] - lo)) | (to_tree ? COL_TREE : 0u));
                    }
                }
            } else {
                constexpr int BOXZ = G::TZ >= 2 ? 2 : 1;         // a flat tile sees one z-slice of the coarser particle
                const int z = a.z0 - G::HZ + rz, x = a.x0 - G::HX + rx;
                const int ya = 2 * yy[g], yb = ya + 1;
                // all cells of the coarser particle inside this tile exist (wave-uniform in z and x)
                const bool rows_full = (BOXZ == 1 || (z | 1) < a.zn) && (x | 1) < a.xn;
                const bool first_row = (BOXZ == 1 || (z & 1) == 0) && (x & 1) == 0;
                const bool ina = in && ya >= y0 && ya < y0 + G::TY;
                const bool pooled = a.pool && rows_full && yb < yn;
                const bool keep = pooled || !a.skip_faces;
                const bool oa = ina && keep && (!pooled || first_row);
                const bool ob = in && keep && !pooled && yb >= y0 && yb < y0 + G::TY && yb < yn;
                const unsigned long long ma = __ballot(oa), mb = __ballot(ob);
                if (ma | mb) {
                    int base = 0;
                    const int n_pooled = __popcll(__ballot(oa && pooled));
                    if (lane == 0) {
                        base = atomicAdd(&sh.ncol, __popcll(ma) + __popcll(mb));
                        if (n_pooled) atomicAdd(&sh.nbox, n_pooled);
                    }
                    base = __shfl(base, 0);
                    if (oa) {
                        const int rank = __popcll(ma & below_me);
                        sh.col_idx[base + rank] = i;
                        sh.col_pos[base + rank] = (unsigned short)((r * G::RS + (ya - lo)) | (pooled ? COL_BOX : 0u));
                    }
                    if (ob) {
                        const int rank = __popcll(ma) + __popcll(mb & below_me);
                        sh.col_idx[base + rank] = i;
                        sh.col_pos[base + rank] = (unsigned short)(r * G::RS + (yb - lo));
                    }
                }
            }
        }
    }
}

template <class G, typename T>
__device__ __forceinline__ void scan_window_dx(const ConvArgs<T>& a, int L, int z0, int x0, int y0, bool out_tree,
                                               ConvShared<G>& sh, bool pool = true) {
    ScanArgs s;
    s.apr_y = a.apr.y; s.tree_y = a.tree.y; s.tree_off = (int)a.tree_off; s.yn = a.apr.y_num[L]; s.y0 = y0;
    s.tree_from_x = (L == a.Lc); s.out_tree = out_tree;
    s.z0 = z0; s.x0 = x0; s.zn = a.apr.z_num[L]; s.xn = a.apr.x_num[L]; s.pool = pool;
    s.skip_faces = pool && a.dx_skip_faces != 0;
    scan_window_dx_impl<G>(s, sh);
}

// End of a window: reset the list lengths (call between two barriers).
template <class G>
__device__ __forceinline__ void close_window(ConvShared<G>& sh) {
    if (threadIdx.x == 0) { sh.ncol = 0; sh.nitem = 0; sh.nbox = 0; }
}

// Buffer loads: the channel plane is described by a wave-uniform resource (base, size in bytes), the lane
// supplies a 32-bit byte offset, and an offset outside the plane returns zero without touching memory.
// That keeps the address registers to one per item and makes every predicate of the gather (item
// exists / value lives in the tree buffer / channel exists) an out-of-range offset or an empty plane
// instead of a branch.  The entry points refuse channel planes of 4 GiB or more so that offsets fit 32 bits.
constexpr unsigned BUF_OOB = 0xffffffffu;

template <typename T> struct RawLoad;
template <> struct RawLoad<float> {
    typedef int raw;
    static __device__ __forceinline__ raw ld(__amdgpu_buffer_rsrc_t r, unsigned off) { return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0); }
    static __device__ __forceinline__ float cast(raw v) { return __builtin_bit_cast(float, v); }
};
template <> struct RawLoad<bf16_t> {      // 16-bit load, zero-extended; the value is the upper half of an fp32
    typedef int raw;
    static __device__ __forceinline__ raw ld(__amdgpu_buffer_rsrc_t r, unsigned off) { return (int)__builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0); }
    static __device__ __forceinline__ float cast(raw v) { return __builtin_bit_cast(float, v << 16); }
};
template <> struct RawLoad<double> {
    typedef int raw __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ raw ld(__amdgpu_buffer_rsrc_t r, unsigned off) { return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0); }
    static __device__ __forceinline__ double cast(raw v) { return __builtin_bit_cast(double, v); }
};

template <typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t plane_rsrc(const T* base, int64_t ld, int c, int C, int64_t count) {
    const int bytes = c < C ? (int)(count * (int64_t)sizeof(T)) : 0;      // a channel beyond C reads as zeros
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base + (int64_t)c * ld), 0, bytes, 0x00020000);
}

// Values of one channel chunk for the items of this thread, in registers.  Thread t owns items t, t + NT, ...
// ("rounds"); NR of the rounds are held at a time (all of them by default).
template <class G, typename T, int CIB, int NR = (G::MAXITEM + G::NT - 1) / G::NT>
struct ItemRegs {
    static constexpr int ROUNDS = (G::MAXITEM + G::NT - 1) / G::NT;  // items per thread
    static constexpr int IPT = NR;
    typename RawLoad<T>::raw v[IPT][CIB];
    unsigned off[IPT];                 // byte offset of the item inside a channel plane (BUF_OOB: no item)
    unsigned short pos[IPT];           // patch cell and flags (0xffff: no item)
};

// Issues the loads of a chunk (no LDS writes: they may run ahead of the consumer of the patch).
// Thread t owns items t, t + NT, ...; a round k that lies beyond the item count is skipped by a
// wave-uniform branch (most windows hold fewer items than the block has threads).
// Which items this thread stages, and where they go: read once per window from the lists (LDS or global).
template <class G, typename T, int CIB, int NR, class Lists>
__device__ __forceinline__ void fetch_slots(const Lists& sh, int nitem, ItemRegs<G, T, CIB, NR>& R, int round0 = 0) {
    if constexpr (std::is_same<Lists, WindowLists>::value) {
        // Lists in global memory: every round is an unconditional buffer load (lanes past the window's items read
        // zero) and nothing is done with the results before all rounds are issued.  A load under a per-lane branch
        // whose result is scaled inside the branch waits for memory there: one round trip per round.
        const __amdgpu_buffer_rsrc_t ri = __builtin_amdgcn_make_buffer_rsrc(const_cast<int*>(sh.item_idx), 0, nitem * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t rp = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned short*>(sh.item_pos), 0, nitem * 2, 0x00020000);
        int idx[NR], pos[NR];
        // the list offsets are formed from this copy of the thread index on every call: kept across the window loop
        // they are spilled, and a reload from scratch before a list load makes that load wait for the one before it
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            idx[k] = 0; pos[k] = 0;
            if ((round0 + k) * G::NT >= nitem) continue;    // wave-uniform
            const int it = tid + (round0 + k) * G::NT;
            idx[k] = __builtin_amdgcn_raw_buffer_load_b32(ri, it * 4, 0, 0);
            pos[k] = (int)__builtin_amdgcn_raw_buffer_load_b16(rp, it * 2, 0, 0);
        }
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            const bool valid = (int)threadIdx.x + (round0 + k) * G::NT < nitem;
            R.pos[k] = valid ? (unsigned short)pos[k] : (unsigned short)0xffffu;
            R.off[k] = valid ? (unsigned)idx[k] * (unsigned)sizeof(T) : BUF_OOB;
        }
    } else {
#pragma unroll
        for (int k = 0; k < NR; ++k) {
            R.pos[k] = 0xffffu; R.off[k] = BUF_OOB;
            if ((round0 + k) * G::NT >= nitem) continue;    // wave-uniform
            const int it = threadIdx.x + (round0 + k) * G::NT;
            if (it < nitem) {
                R.pos[k] = sh.item_pos[it];
                R.off[k] = (unsigned)sh.item_idx[it] * (unsigned)sizeof(T);
            }
        }
    }
}

// Issues the value loads of one chunk for the fetched slots.
// FUSE (a tag argument, so that the other template arguments stay deduced): the kernel was built for the fused
// forward entry points and honours a.x2 / a.c_split; otherwise those fields are not looked at.
template <class G, typename T, int CIB, int NR, bool FUSE = false>
__device__ __forceinline__ void load_values(const ConvArgs<T>& a, int ci0, int nitem, bool tree_items,
                                            ItemRegs<G, T, CIB, NR>& R, int round0 = 0, std::bool_constant<FUSE> = {}) {
    __amdgpu_buffer_rsrc_t rx[CIB], rt[CIB];
#pragma unroll
    for (int c = 0; c < CIB; ++c) {
        const int ch = ci0 + c;
        if (FUSE && a.x2 != nullptr && ch >= a.c_split)
            rx[c] = plane_rsrc<T>(a.x2, a.ldx2, ch - a.c_split, a.Cin - a.c_split, a.x_count);
        else
            rx[c] = plane_rsrc<T>(a.x, a.ldx, ch, a.Cin, a.x_count);
        rt[c] = plane_rsrc<T>(a.tree_data, a.ldt, ci0 + c, tree_items ? a.Cin : 0, a.t_count);
    }
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        if ((round0 + k) * G::NT >= nitem) break;       // wave-uniform
        const bool from_tree = (R.pos[k] & ITEM_TREE) != 0 && R.pos[k] != 0xffffu;
        if (tree_items) {      // tile-uniform: only levels below the current maximum read the mean-filled tree
            // Each lane loads from the one tensor its item lives in, under its own half of the execution mask, into
            // the same registers: no second set of registers and no wait between the two groups of loads (combining
            // two full loads per channel made the compiler wait for every tree load before it issued the next).
            if (from_tree) {
#pragma unroll
                for (int c = 0; c < CIB; ++c) R.v[k][c] = RawLoad<T>::ld(rt[c], R.off[k]);
                asm volatile("" ::: "memory");       // keeps the two branches from being merged into one load with a per-lane descriptor
            } else {
#pragma unroll
                for (int c = 0; c < CIB; ++c) R.v[k][c] = RawLoad<T>::ld(rx[c], R.off[k]);
            }
        } else {
#pragma unroll
            for (int c = 0; c < CIB; ++c) R.v[k][c] = RawLoad<T>::ld(rx[c], R.off[k]);
        }
    }
}

// Issues the loads of a chunk (no LDS writes: they may run ahead of the consumer of the patch).
// Thread t owns items t, t + NT, ...; a round k that lies beyond the item count is skipped by a
// wave-uniform branch (most windows hold fewer items than the block has threads).
template <class G, typename T, int CIB, int NR, class Lists, bool FUSE = false>
__device__ __forceinline__ void load_items(const ConvArgs<T>& a, int ci0, int nitem, bool tree_items,
                                           const Lists& sh, ItemRegs<G, T, CIB, NR>& R, int round0 = 0,
                                           std::bool_constant<FUSE> fuse = {}) {
    fetch_slots<G, T, CIB, NR>(sh, nitem, R, round0);
    load_values<G, T, CIB, NR>(a, ci0, nitem, tree_items, R, round0, fuse);
}

template <class G, typename T, int CIB, int NR>
__device__ __forceinline__ void store_items(const ItemRegs<G, T, CIB, NR>& R, int nitem, typename Num<T>::acc* patch,
                                            int round0 = 0) {
#pragma unroll
    for (int k = 0; k < NR; ++k) {
        if ((round0 + k) * G::NT >= nitem) break;       // wave-uniform
        if (R.pos[k] == 0xffffu) continue;
        typename Num<T>::acc* cell = patch + (R.pos[k] & ITEM_CELL);
#pragma unroll
        for (int c = 0; c < CIB; ++c) {
            const typename Num<T>::acc v = RawLoad<T>::cast(R.v[k][c]);
            cell[c * G::CH_STRIDE] = v;
            if (R.pos[k] & ITEM_PAIR) cell[c * G::CH_STRIDE + 1] = v;
        }
    }
}

// Gather of one channel chunk into the patch.  Cells that no item covers keep the zeros written once
// per window (outside the image, or inside a particle two or more levels coarser, which a stencil of
// half-width <= 2 never reads on a 2:1-balanced APR); covered cells are overwritten by every chunk.
template <class G, typename T, int CIB, bool FUSE = false>
__device__ __forceinline__ void stage_values(const ConvArgs<T>& a, int ci0, int nitem, bool tree_items,
                                             const ConvShared<G>& sh, typename Num<T>::acc* patch,
                                             std::bool_constant<FUSE> fuse = {}) {
    ItemRegs<G, T, CIB> R;
    load_items<G, T, CIB>(a, ci0, nitem, tree_items, sh, R, 0, fuse);
    store_items<G, T, CIB>(R, nitem, patch);
}

}  // namespace aprnet
