// Window lists: what the convolution kernels stage and compute per window, built once per APR, level delta and
// stencil and kept in the plan.  A list entry is an index into the feature / tree vector plus a cell of the LDS
// patch, so the lists depend on the APR alone; every convolution call at that level delta reuses them and its
// kernel neither searches the access arrays nor keeps list bookkeeping in LDS.
//
// Two passes over the tiles with the scanning code of conv_common.hpp: the first counts windows, items and
// columns per tile, the host turns the counts into offsets, the second writes the lists in tile order.
#include "conv_common.hpp"

#include <numeric>

namespace aprnet {

// DX: lists of the input gradient (scan_window_dx without pooled columns) over the tiles within one row of an
// output; windows without an output position are not stored.
//
// Forward lists keep the items that some output position of the window can reach through the stencil.  The scan
// yields every particle and tree node of the staged rows, but a window of a coarser level often holds a handful of
// output positions next to long runs of tree nodes standing for finely resolved regions: no output reads those, so
// they are neither staged by the kernels nor needed in the mean-filled tree (need.hip).
template <class G, bool DX>
__global__ void __launch_bounds__(G::NT)
build_lists_kernel(const ConvArgs<float> a, const int pass, int4* __restrict__ tile_counts, const int4* __restrict__ tile_off,
                   int4* __restrict__ win, int* __restrict__ item_idx, unsigned short* __restrict__ item_pos,
                   int* __restrict__ col_idx, unsigned short* __restrict__ col_pos) {
    __shared__ ConvShared<G> sh;
    __shared__ unsigned char reach[DX ? 4 : G::NROW * G::RS];   // cell -> an output position of its row lies within the y taps
    __shared__ int kept;
    static_assert((G::NROW * G::RS) % 4 == 0, "the reach map is cleared with 4-byte stores");
    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level;
    const int yn = a.apr.y_num[L];
    const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
    int nwin = 0, ni = 0, ncl = 0;
    int4 off = make_int4(0, 0, 0, 0);
    if (pass == 1) off = tile_off[blockIdx.x];

    open_segments<G, float>(a, L, tile.z0, tile.x0, sh);
    __syncthreads();
    for (int y0 = 0; y0 < yn; y0 += G::TY) {
        if constexpr (DX) scan_window_dx<G, float>(a, L, tile.z0, tile.x0, y0, out_tree, sh, false);
        else scan_window<G, float>(a, L, y0, out_tree, sh);
        __syncthreads();
        const int nc = sh.ncol, nitem = sh.nitem;
        if (nc > 0 && (!DX || nitem > 0)) {
            // list offsets are unsigned 32-bit numbers stored in the int fields of the header
            const unsigned ib = (unsigned)off.y + (unsigned)ni, cb = (unsigned)off.z + (unsigned)ncl;
            int nkeep = nitem;
            if constexpr (DX) {
                if (pass == 1)
                    for (int i = threadIdx.x; i < nitem; i += G::NT) { item_idx[(size_t)ib + i] = sh.item_idx[i]; item_pos[(size_t)ib + i] = sh.item_pos[i]; }
            } else {
                for (int i = threadIdx.x; i < G::NROW * G::RS / 4; i += G::NT) reinterpret_cast<int*>(reach)[i] = 0;
                if (threadIdx.x == 0) kept = 0;
                __syncthreads();
                for (int i = threadIdx.x; i < nc; i += G::NT) {
                    const int cell = sh.col_pos[i] & COL_CELL, y = cell % G::RS, row = cell - y;
                    for (int yy = max(y - G::HY, 0); yy <= min(y + G::HY, G::RS - 1); ++yy) reach[row + yy] = 1;
                }
                __syncthreads();
                for (int i0 = 0; i0 < nitem; i0 += G::NT) {
                    const int i = i0 + (int)threadIdx.x;
                    bool keep = false;
                    unsigned pos = 0;
                    if (i < nitem) {
                        pos = sh.item_pos[i];
                        const int cell = pos & 0x0fffu, y = cell % G::RS, r = cell / G::RS, rz = r / G::RX, rx = r - rz * G::RX;
                        const bool pair = (pos & ITEM_PAIR) != 0 && y + 1 < G::RS;
                        for (int dz = -G::HZ; dz <= G::HZ; ++dz)
                            for (int dx = -G::HX; dx <= G::HX; ++dx) {
                                const int z2 = rz + dz, x2 = rx + dx;
                                if (z2 < 0 || z2 >= G::RZ || x2 < 0 || x2 >= G::RX) continue;
                                const int c2 = (z2 * G::RX + x2) * G::RS + y;
                                keep = keep || reach[c2] != 0 || (pair && reach[c2 + 1] != 0);
                            }
                    }
                    const unsigned long long m = __ballot(keep);
                    int base = 0;
                    if (lane_id() == 0 && m) base = atomicAdd(&kept, __popcll(m));
                    base = __shfl(base, 0);
                    if (keep && pass == 1) {
                        const size_t dst = (size_t)ib + base + __popcll(m & ((1ull << lane_id()) - 1ull));
                        item_idx[dst] = sh.item_idx[i]; item_pos[dst] = (unsigned short)pos;
                    }
                }
                __syncthreads();
                nkeep = kept;
            }
            if (pass == 1) {
                if (threadIdx.x == 0) win[off.x + nwin] = make_int4((int)ib, nkeep, (int)cb, nc);
                for (int i = threadIdx.x; i < nc; i += G::NT) { col_idx[(size_t)cb + i] = sh.col_idx[i]; col_pos[(size_t)cb + i] = sh.col_pos[i]; }
            }
            ++nwin; ni += nkeep; ncl += nc;
        }
        __syncthreads();
        close_window<G>(sh);
        __syncthreads();
    }
    if (pass == 0 && threadIdx.x == 0) tile_counts[blockIdx.x] = make_int4(nwin, ni, ncl, 0);
}

using L333 = ConvGeom<3, 3, 3, 2, 4, 512>;
using L133 = ConvGeom<1, 3, 3, 1, 8, 512>;
using L155 = ConvGeom<1, 5, 5, 1, 8, 512>;

template <class G>
static void launch_build(const ConvArgs<float>& a, int n_tiles, int pass, int4* counts, const int4* offs, const WinLists& wl,
                         bool dx, hipStream_t st) {
    if (dx)
        hipLaunchKernelGGL((build_lists_kernel<G, true>), dim3((unsigned)n_tiles), dim3(G::NT), 0, st, a, pass, counts, offs,
                           wl.d_win, wl.d_item_idx, wl.d_item_pos, wl.d_col_idx, wl.d_col_pos);
    else
        hipLaunchKernelGGL((build_lists_kernel<G, false>), dim3((unsigned)n_tiles), dim3(G::NT), 0, st, a, pass, counts, offs,
                           wl.d_win, wl.d_item_idx, wl.d_item_pos, wl.d_col_idx, wl.d_col_pos);
}

static void launch_build_code(int code, const ConvArgs<float>& a, int n_tiles, int pass, int4* counts, const int4* offs,
                              const WinLists& wl, bool dx, hipStream_t st) {
    if (code == 333) launch_build<L333>(a, n_tiles, pass, counts, offs, wl, dx, st);
    else if (code == 133) launch_build<L133>(a, n_tiles, pass, counts, offs, wl, dx, st);
    else launch_build<L155>(a, n_tiles, pass, counts, offs, wl, dx, st);
}

void free_lists(WinLists& wl) {
    for (void* q : {(void*)wl.d_tile_win, (void*)wl.d_win, (void*)wl.d_item_idx, (void*)wl.d_item_pos, (void*)wl.d_col_idx,
                    (void*)wl.d_col_pos})
        if (q) (void)hipFree(q);
    wl = WinLists{};
}

// Lists of the forward convolution at `level_delta` for stencil `code` (333, 133, 155); `tl` must be the tile list
// of the same stencil.  Built on first use (synchronises the stream and allocates), then served from the plan.
// dx: the lists of the input gradient instead; `tl` is then the tile list with a halo of one row.
int get_lists(aprnet_plan* p, int level_delta, int code, const TileList& tl, WinLists* out, hipStream_t st, bool dx) {
    auto key = std::make_pair(level_delta, code + (dx ? 1000 : 0));
    auto it = p->lists.find(key);
    if (it != p->lists.end()) {
        *out = it->second;
        return it->second.unavailable ? fail(APRNET_ERR_UNSUPPORTED, "window lists are not available for this plan") : 0;
    }
    if (stream_is_capturing(st))
        return fail(APRNET_ERR_UNSUPPORTED, "window lists are built on the first call at a level delta (allocates and synchronises): "
                                            "run it once before capturing the stream");
    WinLists wl{};
    WinLists none{}; none.unavailable = true;
    p->lists[key] = none;             // replaced below when the build succeeds
    if (tl.n > 0) {
        ConvArgs<float> a{};
        a.apr = p->dapr; a.tree = p->dtree; a.tiles = tl.d_tiles; a.Lc = p->lc(level_delta); a.tree_off = p->tree_offset(a.Lc);
        int4* d_counts = nullptr; int4* d_offs = nullptr;
        APRNET_HIP_CHECK(hipMalloc((void**)&d_counts, (size_t)tl.n * sizeof(int4)));
        launch_build_code(code, a, tl.n, 0, d_counts, nullptr, wl, dx, st);
        APRNET_LAUNCH_CHECK("build_lists_kernel (count)");
        std::vector<int4> counts(tl.n), offs(tl.n);
        APRNET_HIP_CHECK(hipStreamSynchronize(st));
        APRNET_HIP_CHECK(hipMemcpy(counts.data(), d_counts, (size_t)tl.n * sizeof(int4), hipMemcpyDeviceToHost));
        std::vector<int> tile_win(tl.n + 1);
        int64_t nw = 0, ni = 0, nc = 0;
        for (int t = 0; t < tl.n; ++t) {
            offs[t] = make_int4((int)nw, (int)(uint32_t)ni, (int)(uint32_t)nc, 0);
            tile_win[t] = (int)nw;
            nw += counts[t].x; ni += counts[t].y; nc += counts[t].z;
        }
        tile_win[tl.n] = (int)nw;
        if (ni >= (int64_t)UINT32_MAX || nc >= (int64_t)UINT32_MAX || nw >= (int64_t)INT32_MAX) {
            (void)hipFree(d_counts);
            return fail(APRNET_ERR_UNSUPPORTED, "window lists: more than 2^32 entries");
        }
        wl.n_win = (int)nw; wl.n_items = ni; wl.n_cols = nc;
        for (int l = MAX_LEVELS; l >= 0; --l) {        // tiles are sorted finest level first
            if (tl.level_count[l] <= 0) continue;
            const int fw = tile_win[tl.level_begin[l]], lw = tile_win[tl.level_begin[l] + tl.level_count[l]];
            if (lw > fw) { wl.lv_first[wl.n_lv] = fw; wl.lv_level[wl.n_lv] = l; ++wl.n_lv; }
        }
        auto alloc = [&](void** q, size_t bytes) -> int { APRNET_HIP_CHECK(hipMalloc(q, std::max<size_t>(bytes, 16))); return 0; };
        int rc = alloc((void**)&d_offs, (size_t)tl.n * sizeof(int4));
        if (!rc) rc = alloc((void**)&wl.d_tile_win, tile_win.size() * sizeof(int));
        if (!rc) rc = alloc((void**)&wl.d_win, (size_t)nw * sizeof(int4));
        if (!rc) rc = alloc((void**)&wl.d_item_idx, (size_t)ni * sizeof(int));
        if (!rc) rc = alloc((void**)&wl.d_item_pos, (size_t)ni * sizeof(unsigned short));
        if (!rc) rc = alloc((void**)&wl.d_col_idx, (size_t)nc * sizeof(int));
        if (!rc) rc = alloc((void**)&wl.d_col_pos, (size_t)nc * sizeof(unsigned short));
        if (rc) { (void)hipFree(d_counts); if (d_offs) (void)hipFree(d_offs); free_lists(wl); return rc; }
        APRNET_HIP_CHECK(hipMemcpy(d_offs, offs.data(), (size_t)tl.n * sizeof(int4), hipMemcpyHostToDevice));
        APRNET_HIP_CHECK(hipMemcpy(wl.d_tile_win, tile_win.data(), tile_win.size() * sizeof(int), hipMemcpyHostToDevice));
        launch_build_code(code, a, tl.n, 1, d_counts, d_offs, wl, dx, st);
        APRNET_LAUNCH_CHECK("build_lists_kernel (fill)");
        APRNET_HIP_CHECK(hipStreamSynchronize(st));
        (void)hipFree(d_counts); (void)hipFree(d_offs);
    }
    p->lists[key] = wl;
    *out = wl;
    return 0;
}

}  // namespace aprnet
