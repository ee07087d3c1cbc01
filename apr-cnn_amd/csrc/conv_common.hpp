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

namespace aprnet {

template <typename T>
struct ConvArgs {
    AccessDev apr, tree;
    const ConvTile* tiles;
    const T* x; int64_t ldx; int Cin;
    const T* w; int S_exp; int Cout;          // [S_exp][Cout][Cin][K]
    T* y; int64_t ldy;
    const T* tree_data; int64_t ldt;
    int Lc; int64_t tree_off;                  // tree_offset(Lc)
    // backward only
    const T* gy; T* gx; int64_t ldgx; T* gtree; int64_t ldgt; T* gw; int n_tiles;
};

template <int KZ_, int KX_, int KY_, int TZ_, int TX_, int NT_>
struct ConvGeom {
    static constexpr int KZ = KZ_, KX = KX_, KY = KY_, TZ = TZ_, TX = TX_, NT = NT_;
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
    static constexpr int ITER = (MAXCOL + NT - 1) / NT;        // output columns per thread
    static constexpr int CH_STRIDE = NROW * WY;                // patch elements per channel
    static constexpr int TAP0 = (HZ * RX + HX) * WY + HY;      // centre -> first tap
};

__device__ __forceinline__ int lane_id() { return __lane_id(); }

// Per-block bookkeeping kept in LDS.
template <class G>
struct ConvShared {
    int seg_cur[G::NSEG];            // cursor: first particle of the segment that can fall into the current window
    int seg_end[G::NSEG];
    int seg_next[G::NSEG];           // cursor for the next window
    unsigned char seg_nin[G::NSEG];  // particles of the segment inside the current window (a prefix of the 64 lanes)
    int col_idx[G::MAXCOL];          // output positions of the window: feature index ...
    unsigned short col_pos[G::MAXCOL];   // ... and centre cell inside one channel of the patch
    int ncol;
};

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

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
    if (threadIdx.x == 0) sh.ncol = 0;
}

// Phase A of a window.  Every wave loads y_vec at the cursor of its segments (64 lanes = every particle
// that can fall into the 64-cell window), and from ballots over "y < bound" derives the number of
// in-window particles (they are the first n lanes, y ascends) and the cursor of the next window.
// Particles of the centre rows (plus tree nodes when they are downsampled particles) whose y lies in the
// output range are appended to the column list.
template <class G, typename T>
__device__ __forceinline__ void scan_window(const ConvArgs<T>& a, int L, int y0, bool out_tree, ConvShared<G>& sh) {
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int lo = y0 - G::HY, hi = y0 + G::TY + G::HY, lo_next = y0 + G::TY - G::HY;
#pragma unroll 6
    for (int k = 0; k < G::SPW; ++k) {
        const int s = wave + k * G::NWAVE;
        if (s >= G::NSEG) break;
        const int r = s / 3, src = s - 3 * r;
        const int cur = sh.seg_cur[s];
        const int i = cur + lane;
        const bool valid = i < sh.seg_end[s];
        int yy = INT_MAX;
        if (valid) yy = (src == 2) ? (int)a.tree.y[i] : (int)a.apr.y[i];
        const bool in = valid && (src == 1 ? yy <= ((hi - 1) >> 1) : yy < hi);
        const bool below = valid && (src == 1 ? yy < (lo_next >> 1) : yy < lo_next);
        const int n_in = __popcll(__ballot(in)), n_adv = __popcll(__ballot(below));
        if (lane == 0) { sh.seg_nin[s] = (unsigned char)n_in; sh.seg_next[s] = cur + n_adv; }
        const int rz = r / G::RX, rx = r - rz * G::RX;
        const bool centre = rz >= G::HZ && rz < G::HZ + G::TZ && rx >= G::HX && rx < G::HX + G::TX;
        const bool out_seg = centre && (src == 0 || (src == 2 && out_tree));
        const bool outl = out_seg && in && yy >= y0 && yy < y0 + G::TY;
        const unsigned long long m = __ballot(outl);
        if (m) {
            int base = 0;
            if (lane == 0) base = atomicAdd(&sh.ncol, __popcll(m));
            base = __shfl(base, 0);
            if (outl) {
                const int rank = __popcll(m & ((1ull << lane) - 1ull));
                sh.col_idx[base + rank] = i + (src == 2 ? (int)a.tree_off : 0);
                sh.col_pos[base + rank] = (unsigned short)(r * G::WY + (yy - lo));
            }
        }
    }
}

// Phase C: commit the cursors of the next window.
template <class G>
__device__ __forceinline__ void advance_cursors(ConvShared<G>& sh) {
    for (int s = threadIdx.x; s < G::NSEG; s += G::NT) sh.seg_cur[s] = sh.seg_next[s];
    if (threadIdx.x == 0) sh.ncol = 0;
}

// Walks the in-window particles of the wave's segments: f(r, src, i, yy) per lane that holds one.
// The y of a particle is re-read here (it is hot in the cache) instead of being kept in registers
// between the phases; the value loads do not depend on it, so both are issued together.
template <class G, typename T, class F>
__device__ __forceinline__ void for_window_particles(const ConvArgs<T>& a, const ConvShared<G>& sh, F f) {
    const int wave = threadIdx.x >> 6, lane = lane_id();
#pragma unroll 6
    for (int k = 0; k < G::SPW; ++k) {
        const int s = wave + k * G::NWAVE;
        if (s >= G::NSEG) break;
        if (lane < (int)sh.seg_nin[s]) {
            const int r = s / 3, src = s - 3 * r;
            const int i = sh.seg_cur[s] + lane;
            const int yy = (src == 2) ? (int)a.tree.y[i] : (int)a.apr.y[i];
            f(r, src, i, yy);
        }
    }
}

// Gather of one channel chunk into the (already zeroed) patch.
template <class G, typename T, int CIB>
__device__ __forceinline__ void stage_values(const ConvArgs<T>& a, int L, int y0, int ci0, const ConvShared<G>& sh,
                                             T* patch) {
    const int lo = y0 - G::HY, hi = y0 + G::TY + G::HY;
    const int yn = a.apr.y_num[L];
    const bool tree_from_x = (L == a.Lc);
    for_window_particles<G, T>(a, sh, [&](int r, int src, int i, int yy) {
        const T* base;
        int64_t ld;
        if (src == 2 && !tree_from_x) { base = a.tree_data + i; ld = a.ldt; }
        else { base = a.x + i + (src == 2 ? a.tree_off : 0); ld = a.ldx; }
        T v[CIB];
#pragma unroll
        for (int c = 0; c < CIB; ++c) v[c] = (ci0 + c < a.Cin) ? base[(int64_t)(ci0 + c) * ld] : (T)0;
        T* prow = patch + r * G::WY;
        if (src != 1) {
#pragma unroll
            for (int c = 0; c < CIB; ++c) prow[c * G::CH_STRIDE + (yy - lo)] = v[c];
        } else {
            const int ya = 2 * yy, yb = ya + 1;
            const bool wa = ya >= lo && ya < hi, wb = yb >= lo && yb < hi && yb < yn;
#pragma unroll
            for (int c = 0; c < CIB; ++c) {
                if (wa) prow[c * G::CH_STRIDE + (ya - lo)] = v[c];
                if (wb) prow[c * G::CH_STRIDE + (yb - lo)] = v[c];
            }
        }
    });
}

}  // namespace aprnet
