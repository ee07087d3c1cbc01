// Stencil convolution, backward: Convolution<kz,kx,ky>::backward (conv.hpp:261-481 with
// helpers.hpp:423-478, 578-704).  Two kernels over the same tiles / windows as the forward pass.
//
// grad_input.  Per window and chunk of input channels every thread owns one output position and
// forms its K tap gradients  g[c][t] = sum_co dO[co] * w[co][c][t]  (weights wave-uniform), adds
// them into an LDS gradient patch (LDS atomics: neighbouring outputs overlap), and the patch is then
// flushed along the three gather sources - the exact transpose of the forward gather, including the
// two cells of a coarser particle.  Halo rows belong to neighbouring tiles as well, so the flush uses
// global floating-point atomics; tree cells of levels < Lc go to the tree-gradient buffer that
// fill_tree_mean_backward afterwards pushes down to the particles.
//
// grad_weights.  dW[s][co][ci][t] = sum over outputs of dO[co] * tap[ci][t].  A thread owns one
// (co, ci) pair and keeps its K sums in registers while the (persistent) block walks over many
// tiles; dO and the patch are staged in LDS.  Sums are flushed with one atomic per element when the
// stencil index changes and at the end.
#include "conv_common.hpp"

namespace aprnet {

template <typename T>
__global__ void fill_kernel(T* __restrict__ p, int64_t ld, int64_t n, T v) {
    T* row = p + (int64_t)blockIdx.y * ld;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) row[i] = v;
}

template <typename T>
static void fill2d(T* p, int64_t ld, int64_t n, int rows, T v, hipStream_t st) {
    if (n <= 0 || rows <= 0) return;
    dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 4096), (unsigned)rows);
    hipLaunchKernelGGL(fill_kernel<T>, grid, dim3(256), 0, st, p, ld, n, v);
}

// Transpose of stage_values: add the gradient patch back to its sources, item by item.
template <class G, typename T, int CIB>
__device__ __forceinline__ void flush_values(const ConvArgs<T>& a, int ci0, int nitem, const ConvShared<G>& sh,
                                             const T* gpatch) {
    for (int it = threadIdx.x; it < nitem; it += G::NT) {
        const unsigned pos = sh.item_pos[it];
        const int64_t idx = sh.item_idx[it];
        T* base = (pos & ITEM_TREE) ? a.gtree + idx : a.gx + idx;
        const int64_t ld = (pos & ITEM_TREE) ? a.ldgt : a.ldgx;
        const T* cell = gpatch + (pos & ITEM_CELL);
#pragma unroll
        for (int c = 0; c < CIB; ++c) {
            if (ci0 + c >= a.Cin) break;
            T v = cell[c * G::CH_STRIDE];
            if (pos & ITEM_PAIR) v += cell[c * G::CH_STRIDE + 1];
            if (v != (T)0) atomicAdd(base + (int64_t)(ci0 + c) * ld, v);
        }
    }
}

template <typename T, class G, int CIB, int COBLK>
__global__ void __launch_bounds__(G::NT)
conv_bwd_dx_kernel(const ConvArgs<T> a) {
    static_assert(G::ITER == 1, "one output position per thread");
    __shared__ T gpatch[CIB * G::CH_STRIDE];
    __shared__ T dOs[COBLK * G::MAXCOL];
    __shared__ ConvShared<G> sh;

    const ConvTile tile = a.tiles[blockIdx.x];
    const int L = tile.level, z0 = tile.z0, x0 = tile.x0;
    const int ci0 = blockIdx.y * CIB;
    const int yn = a.apr.y_num[L];
    const int s_idx = min(a.S_exp - 1, a.Lc - L);
    const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
    const T* __restrict__ wl = a.w + (int64_t)s_idx * a.Cout * a.Cin * G::K;

    open_segments<G, T>(a, L, z0, x0, sh);
    __syncthreads();

    for (int y0 = 0; y0 < yn; y0 += G::TY) {
        scan_window<G, T>(a, L, y0, out_tree, sh);
        __syncthreads();
        const int nc = sh.ncol, nitem = sh.nitem;
        if (nc > 0) {
            for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) gpatch[i] = 0;
            T g[CIB][G::K];
#pragma unroll
            for (int c = 0; c < CIB; ++c)
#pragma unroll
                for (int t = 0; t < G::K; ++t) g[c][t] = 0;
            const int col = threadIdx.x;
            for (int co0 = 0; co0 < a.Cout; co0 += COBLK) {
                __syncthreads();
                const int nco = min(COBLK, a.Cout - co0);
                for (int i = threadIdx.x; i < nco * nc; i += G::NT) {
                    const int co = i / nc, cc = i - co * nc;
                    dOs[co * G::MAXCOL + cc] = a.gy[(int64_t)(co0 + co) * a.ldy + sh.col_idx[cc]];
                }
                __syncthreads();
                if (col < nc) {
#pragma unroll 1
                    for (int co = 0; co < nco; ++co) {
                        const T dO = dOs[co * G::MAXCOL + col];
#pragma unroll
                        for (int c = 0; c < CIB; ++c) {
                            if (ci0 + c >= a.Cin) break;
                            const T* __restrict__ wp = wl + ((int64_t)(co0 + co) * a.Cin + ci0 + c) * G::K;
#pragma unroll
                            for (int t = 0; t < G::K; ++t) g[c][t] += dO * wp[t];
                        }
                    }
                }
            }
            if (col < nc) {
                T* p0 = gpatch + (int)sh.col_pos[col] - G::TAP0;
#pragma unroll
                for (int c = 0; c < CIB; ++c)
#pragma unroll
                    for (int sz = 0; sz < G::KZ; ++sz)
#pragma unroll
                        for (int sx = 0; sx < G::KX; ++sx)
#pragma unroll
                            for (int sy = 0; sy < G::KY; ++sy)
                                atomicAdd(&p0[c * G::CH_STRIDE + (sz * G::RX + sx) * G::RS + sy],
                                          g[c][(sz * G::KX + sx) * G::KY + sy]);
            }
            __syncthreads();
            flush_values<G, T, CIB>(a, ci0, nitem, sh, gpatch);
        }
        __syncthreads();
        close_window<G>(sh);
        __syncthreads();
    }
}

template <typename T, class G, int CIB, int COB>
__global__ void __launch_bounds__(G::NT)
conv_bwd_dw_kernel(const ConvArgs<T> a) {
    static_assert(CIB * COB <= G::NT, "one thread per (co, ci) pair");
    constexpr int DOS_LD = COB + 1;
    __shared__ T patch[CIB * G::CH_STRIDE];
    __shared__ T dOs[G::MAXCOL * DOS_LD];
    __shared__ ConvShared<G> sh;

    const int ci0 = blockIdx.y * CIB, co0 = blockIdx.z * COB;
    const int pco = threadIdx.x % COB, pc = threadIdx.x / COB;
    const bool worker = threadIdx.x < CIB * COB && (co0 + pco) < a.Cout && (ci0 + pc) < a.Cin;
    T acc[G::K];
#pragma unroll
    for (int t = 0; t < G::K; ++t) acc[t] = 0;
    int cur_s = -1;

    auto flush = [&](int s_idx) {
        if (!worker || s_idx < 0) return;
        T* dst = a.gw + (((int64_t)s_idx * a.Cout + co0 + pco) * a.Cin + ci0 + pc) * G::K;
#pragma unroll
        for (int t = 0; t < G::K; ++t) { if (acc[t] != (T)0) atomicAdd(dst + t, acc[t]); acc[t] = 0; }
    };

    for (int ti = blockIdx.x; ti < a.n_tiles; ti += gridDim.x) {
        const ConvTile tile = a.tiles[ti];
        const int L = tile.level, z0 = tile.z0, x0 = tile.x0;
        const int yn = a.apr.y_num[L];
        const int s_idx = min(a.S_exp - 1, a.Lc - L);
        const bool out_tree = (L == a.Lc) && (L < a.apr.level_max);
        if (s_idx != cur_s) { flush(cur_s); cur_s = s_idx; }

        __syncthreads();
        open_segments<G, T>(a, L, z0, x0, sh);
        __syncthreads();

        for (int y0 = 0; y0 < yn; y0 += G::TY) {
            scan_window<G, T>(a, L, y0, out_tree, sh);
            __syncthreads();
            const int nc = sh.ncol, nitem = sh.nitem;
            if (nc > 0) {
                for (int i = threadIdx.x; i < CIB * G::CH_STRIDE; i += G::NT) patch[i] = 0;
                const int nco = min(COB, a.Cout - co0);
                for (int i = threadIdx.x; i < nco * nc; i += G::NT) {
                    const int co = i / nc, cc = i - co * nc;
                    dOs[cc * DOS_LD + co] = a.gy[(int64_t)(co0 + co) * a.ldy + sh.col_idx[cc]];
                }
                __syncthreads();
                stage_values<G, T, CIB>(a, ci0, nitem, L < a.Lc, sh, patch);
                __syncthreads();
                if (worker) {
                    const T* pch = patch + pc * G::CH_STRIDE - G::TAP0;
                    for (int col = 0; col < nc; ++col) {
                        const T dO = dOs[col * DOS_LD + pco];
                        const T* p0 = pch + (int)sh.col_pos[col];
#pragma unroll
                        for (int sz = 0; sz < G::KZ; ++sz)
#pragma unroll
                            for (int sx = 0; sx < G::KX; ++sx)
#pragma unroll
                                for (int sy = 0; sy < G::KY; ++sy)
                                    acc[(sz * G::KX + sx) * G::KY + sy] += dO * p0[(sz * G::RX + sx) * G::RS + sy];
                    }
                }
            }
            __syncthreads();
            close_window<G>(sh);
            __syncthreads();
        }
    }
    flush(cur_s);
}

// geometries: 512 threads for grad_input (one output position per thread), 256 for grad_weights
using X333 = ConvGeom<3, 3, 3, 2, 4, 512>;
using X133 = ConvGeom<1, 3, 3, 1, 8, 512>;
using X155 = ConvGeom<1, 5, 5, 1, 8, 512>;
using X555 = ConvGeom<5, 5, 5, 2, 4, 512>;
using W333 = ConvGeom<3, 3, 3, 2, 4, 256>;
using W133 = ConvGeom<1, 3, 3, 1, 8, 256>;
using W155 = ConvGeom<1, 5, 5, 1, 8, 256>;
using W555 = ConvGeom<5, 5, 5, 2, 4, 256>;

int fill_tree_for_conv(const aprnet_plan* p, int d, const float* x, int64_t ldx, int C, float* tree, int64_t ldt, hipStream_t st, const NeedLists* need);
int fill_tree_for_conv(const aprnet_plan* p, int d, const double* x, int64_t ldx, int C, double* tree, int64_t ldt, hipStream_t st, const NeedLists* need);
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, float* gx, int64_t ldx, int C, float* gt, int64_t ldt, hipStream_t st);
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, double* gx, int64_t ldx, int C, double* gt, int64_t ldt, hipStream_t st);

template <typename T, class GX, int XCIB, class GW, int WCIB, int WCOB>
static int launch_bwd(ConvArgs<T>& a, hipStream_t st) {
    constexpr int COBLK = 8;
    if (a.gx) {
        dim3 gx((unsigned)a.n_tiles, (unsigned)((a.Cin + XCIB - 1) / XCIB));
        hipLaunchKernelGGL((conv_bwd_dx_kernel<T, GX, XCIB, COBLK>), gx, dim3(GX::NT), 0, st, a);
        APRNET_LAUNCH_CHECK("conv_bwd_dx_kernel");
    }
    dim3 gw((unsigned)std::min(a.n_tiles, 512), (unsigned)((a.Cin + WCIB - 1) / WCIB), (unsigned)((a.Cout + WCOB - 1) / WCOB));
    hipLaunchKernelGGL((conv_bwd_dw_kernel<T, GW, WCIB, WCOB>), gw, dim3(GW::NT), 0, st, a);
    APRNET_LAUNCH_CHECK("conv_bwd_dw_kernel");
    return 0;
}

// matrix-core kernels (conv_mfma.hip, conv_bwd_mfma.hip)
bool conv_mfma_supported(int code);
int launch_conv_dx_mfma(int code, const ConvArgs<float>& a, int n_tiles, hipStream_t st);
int launch_conv_dw_mfma(int code, const ConvArgs<float>& a, const TileList& tl, int level_min, hipStream_t st);
int launch_conv_dx_mfma(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st);
int launch_conv_dw_mfma(int code, const ConvArgs<bf16_t>& a, const TileList& tl, int level_min, hipStream_t st);
int fill_tree_for_conv(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int C, bf16_t* tree, int64_t ldt, hipStream_t st, const NeedLists* need);
size_t conv_packed_floats(int code, int S_exp, int Cm, int Ck, bool transposed);
int pack_conv_weights(int code, const float* w, int S_exp, int Cm, int Ck, bool transposed, float* packed, hipStream_t st);
int conv_path();
// points a at the plan's window lists (conv.hip); leaves a.tile_win null when they are off or unavailable
int set_conv_lists(aprnet_plan* p, int d, int code, const TileList& tl, ConvArgs<float>& a, hipStream_t st);
int set_conv_lists(aprnet_plan* p, int d, int code, const TileList& tl, ConvArgs<bf16_t>& a, hipStream_t st);
int set_conv_dx_lists(aprnet_plan* p, int d, int code, const TileList& tl, ConvArgs<bf16_t>& a, hipStream_t st);
int launch_conv_dx_mfma_bf16(int code, const ConvArgs<bf16_t>& a, int n_tiles, hipStream_t st);
size_t conv_packed_bf16_bytes(int code, int S_exp, int Cout, int Cin);
int pack_conv_weights_bf16(int code, const float* w, int S_exp, int Cout, int Cin, void* packed, hipStream_t st, bool transposed);
int interleave8_bf16(const bf16_t* x, int64_t ldx, const bf16_t* x2, int64_t ldx2, int c_split, int C, int64_t count, bf16_t* out,
                     hipStream_t st);
int bf16_regroup();
int bf16_math();
int bwd_deterministic();
int launch_face_dx(const FaceLists& fl, const float* gy, int64_t ldy, const float* w, int S_exp, int Cout, int Cin, int K, int Lc,
                   float* gx, int64_t ldgx, hipStream_t st);
int conv_dw_partial_blocks(int code, int Cout, int Cin);
size_t conv_dw_partial_bytes(int code, int Cout, int Cin);
// Points the weight-gradient kernels at their partial-sum slots, `off` bytes into the plan's scratch buffer (behind
// whatever the input gradient keeps there: the two run side by side).
template <typename T>
static void set_dw_partials(aprnet_plan* p, size_t off, int code, ConvArgs<T>& a) {
    a.gw_part = (float*)((char*)p->d_scratch + off);
    a.gw_part_ld = (int64_t)a.Cout * a.Cin * (code == 333 ? 27 : code == 133 ? 9 : 25);
    a.gw_part_blocks = conv_dw_partial_blocks(code, a.Cout, a.Cin);
}

template <typename T> static int try_mfma_bwd(aprnet_plan*, const ConvArgs<T>&, const TileList&, int, int, hipStream_t, bool*) { return 0; }
static int fork_side(aprnet_plan* p, hipStream_t st, hipStream_t* side);
static int join_side(aprnet_plan* p, hipStream_t st, hipStream_t side);
// Joins the side stream on every way out of a backward call, also the failing ones: the caller's stream must not run
// ahead of a weight-gradient kernel that still reads the caller's tensors, and a capture must not end with an open fork.
struct SideJoin {
    aprnet_plan* p; hipStream_t st, side; bool open = true;
    SideJoin(aprnet_plan* p_, hipStream_t st_, hipStream_t side_) : p(p_), st(st_), side(side_) {}
    int join() { open = false; return join_side(p, st, side); }
    ~SideJoin() { if (open) (void)join_side(p, st, side); }
};
template <> int try_mfma_bwd<float>(aprnet_plan* p, const ConvArgs<float>& a, const TileList& tl, int code, int d, hipStream_t st, bool* done) {
    if (conv_path() == 1 || !conv_mfma_supported(code)) return 0;
    *done = true;
    // weight gradient on the side stream (when there is an input gradient to run next to)
    ConvArgs<float> c = a;
    if (int rc = set_conv_lists(p, d, code, tl, c, st)) return rc;
    // everything that can allocate or fail on the host comes before the fork
    TileList near;
    FaceLists faces;
    const bool split_faces = a.gx && bwd_deterministic();
    if (a.gx) if (int rc = get_tiles(p, d, code == 333 ? 2 : 1, code == 333 ? 4 : 8, &near, st, 1)) return rc;
    if (split_faces) if (int rc = get_face_lists(p, d, code, &faces, st)) return rc;
    const size_t wbytes = a.gx ? (conv_packed_floats(code, a.S_exp, a.Cin, a.Cout, true) * sizeof(float) + 255) / 256 * 256 : 0;
    const size_t pbytes = bwd_deterministic() ? conv_dw_partial_bytes(code, a.Cout, a.Cin) : 0;
    ScratchLease lease;          // before the join guard below: its hand-over event is recorded after the join
    if (wbytes + pbytes) if (int rc = lease.acquire(p, wbytes + pbytes, st)) return rc;
    if (pbytes) set_dw_partials(p, wbytes, code, c);
    hipStream_t side = st;
    if (a.gx) if (int rc = fork_side(p, st, &side)) return rc;
    SideJoin guard(p, st, side);
    if (int rc = launch_conv_dw_mfma(code, c, tl, p->apr.level_min, side)) return rc;
    if (a.gx) {
        // input gradient: the forward kernel on the output gradient with the transposed, flipped stencil;
        // every row group within one row of an output takes part
        if (int rc = pack_conv_weights(code, a.w, a.S_exp, a.Cin, a.Cout, true, (float*)p->d_scratch, st)) return rc;
        ConvArgs<float> b = a;
        b.tiles = near.d_tiles; b.n_tiles = near.n;
        b.x = a.gy; b.ldx = a.ldy; b.Cin = a.Cout; b.Cout = a.Cin; b.w = (const float*)p->d_scratch; b.bias = nullptr;
        b.tree_data = nullptr; b.t_count = 0;
        b.dx_skip_faces = split_faces ? 1 : 0;
        if (near.n > 0) if (int rc = launch_conv_dx_mfma(code, b, near.n, st)) return rc;
        // coarser particles with cells outside their finer level: summed pair by pair in list order
        if (split_faces)
            if (int rc = launch_face_dx(faces, a.gy, a.ldy, a.w, a.S_exp, a.Cout, a.Cin, code == 333 ? 27 : code == 133 ? 9 : 25, a.Lc,
                                        a.gx, a.ldgx, st)) return rc;
    }
    return guard.join();
}

// Fork / join around the two halves of the backward pass: what follows fork() on the returned stream runs next to
// the caller's stream `st` until join().  Both kernels are bound by their matrix phases and the barriers between
// them at about half of the matrix peak, and read the same output gradient; side by side they fill each other's
// gaps.  Default priority, event based, so a caller may capture it into a graph.
int backward_overlap();
static int fork_side(aprnet_plan* p, hipStream_t st, hipStream_t* side) {
    *side = st;
    if (!backward_overlap()) return 0;
    if (!p->side) {
        APRNET_HIP_CHECK(hipStreamCreateWithFlags(&p->side, hipStreamNonBlocking));
        APRNET_HIP_CHECK(hipEventCreateWithFlags(&p->ev_fork, hipEventDisableTiming));
        APRNET_HIP_CHECK(hipEventCreateWithFlags(&p->ev_join, hipEventDisableTiming));
    }
    APRNET_HIP_CHECK(hipEventRecord(p->ev_fork, st));
    APRNET_HIP_CHECK(hipStreamWaitEvent(p->side, p->ev_fork, 0));
    *side = p->side;
    return 0;
}
static int join_side(aprnet_plan* p, hipStream_t st, hipStream_t side) {
    if (side == st) return 0;
    APRNET_HIP_CHECK(hipEventRecord(p->ev_join, side));
    APRNET_HIP_CHECK(hipStreamWaitEvent(st, p->ev_join, 0));
    return 0;
}

template <typename T>
int conv_bwd(const aprnet_plan* cp, int d, int kz, int kx, int ky, const T* x, int64_t ldx, int Cin, const T* w, int S_exp,
             int Cout, const T* gy, int64_t ldy, T* gx, int64_t ldgx, T* gw, T* tree_ws, int64_t ldt, T* gtree_ws,
             int64_t ldgt, hipStream_t st) {
    aprnet_plan* p = const_cast<aprnet_plan*>(cp);
    if (int rc = check_level_delta(p, d, "conv_backward")) return rc;
    if (int rc = check_plane_size(p, d, sizeof(*x), "conv_backward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv_backward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv_backward", "output gradient")) return rc;
    if (gx) if (int rc = check_rows(ldgx, p->number_parts(d), "conv_backward", "input gradient")) return rc;
    if (Cin <= 0 || Cout <= 0 || S_exp <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv_backward: empty channel / stencil count");
    const int code = kz * 100 + kx * 10 + ky;
    if (code != 333 && code != 133 && code != 155 && code != 555)
        return fail(APRNET_ERR_UNSUPPORTED, "conv_backward: stencil must be 333, 133, 155 or 555");
    const int64_t nt = p->tree_parts(d);
    // gx == nullptr: the caller does not need the input gradient (first layer of a network); only gw is computed
    if (nt > 0 && (!tree_ws || ldt < nt || (gx && (!gtree_ws || ldgt < nt))))
        return fail(APRNET_ERR_INVALID_ARGUMENT, "conv_backward: tree work space too small");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    if (int rc = fill_tree_for_conv(p, d, x, ldx, Cin, tree_ws, ldt, st, nullptr)) return rc;
    if (gx) {
        fill2d<T>(gx, ldgx, p->number_parts(d), Cin, (T)0, st);
        fill2d<T>(gtree_ws, ldgt, nt, Cin, (T)0, st);
    }
    const bool flat = (kz == 1);
    TileList tl;
    if (int rc = get_tiles(p, d, flat ? 1 : 2, flat ? 8 : 4, &tl, st)) return rc;
    if (tl.n > 0) {
        ConvArgs<T> a{};
        a.apr = p->dapr; a.tree = p->dtree; a.tiles = tl.d_tiles; a.n_tiles = tl.n;
        a.x = x; a.ldx = ldx; a.Cin = Cin; a.w = w; a.S_exp = S_exp; a.Cout = Cout;
        a.tree_data = tree_ws; a.ldt = ldt; a.Lc = p->lc(d); a.tree_off = p->tree_offset(a.Lc);
    a.x_count = p->number_parts(d); a.t_count = p->tree_parts(d);
        a.gy = gy; a.ldy = ldy; a.gx = gx; a.ldgx = ldgx; a.gtree = gtree_ws; a.ldgt = ldgt; a.gw = gw;
        constexpr bool f32 = sizeof(T) == 4;
        int rc = 0;
        bool done = false;
        if ((rc = try_mfma_bwd<T>(p, a, tl, code, d, st, &done))) return rc;
        if (!done) switch (code) {
            case 333: rc = launch_bwd<T, X333, (f32 ? 4 : 2), W333, (f32 ? 8 : 4), (f32 ? 32 : 16)>(a, st); break;
            case 133: rc = launch_bwd<T, X133, (f32 ? 8 : 4), W133, (f32 ? 8 : 4), (f32 ? 32 : 16)>(a, st); break;
            case 155: rc = launch_bwd<T, X155, (f32 ? 4 : 2), W155, (f32 ? 8 : 4), (f32 ? 32 : 16)>(a, st); break;
            case 555: rc = launch_bwd<T, X555, 1, W555, (f32 ? 4 : 2), (f32 ? 32 : 16)>(a, st); break;
        }
        if (rc) return rc;
    }
    return gx ? fill_tree_bwd_for_conv(p, d, gx, ldgx, Cin, gtree_ws, ldgt, st) : 0;
}

__global__ void round_to_bf16_kernel(const float* __restrict__ src, int64_t lds, bf16_t* __restrict__ dst, int64_t ldd, int64_t n) {
    const float* s = src + (int64_t)blockIdx.y * lds;
    bf16_t* d = dst + (int64_t)blockIdx.y * ldd;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) d[i] = float_to_bf16(s[i]);
}

// bfloat16 features and output gradient; weights, weight gradient and all accumulation in fp32 (the fp32
// matrix-core kernels with 16-bit loads).  gx32_ws [Cin][ldgx32] and gtree_ws [Cin][ldgt] are fp32 work space:
// the input gradient is accumulated there and rounded to bfloat16 at the end.
int conv_bwd_bf16(const aprnet_plan* cp, int d, int kz, int kx, int ky, const bf16_t* x, int64_t ldx, int Cin, const float* w,
                  int S_exp, int Cout, const bf16_t* gy, int64_t ldy, bf16_t* gx, int64_t ldgx, float* gw, bf16_t* tree_ws,
                  int64_t ldt, float* gx32_ws, int64_t ldgx32, float* gtree_ws, int64_t ldgt, hipStream_t st) {
    aprnet_plan* p = const_cast<aprnet_plan*>(cp);
    if (int rc = check_level_delta(p, d, "conv_backward")) return rc;
    if (int rc = check_plane_size(p, d, sizeof(float), "conv_backward")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "conv_backward", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv_backward", "output gradient")) return rc;
    if (gx) if (int rc = check_rows(ldgx, p->number_parts(d), "conv_backward", "input gradient")) return rc;
    if (Cin <= 0 || Cout <= 0 || S_exp <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv_backward: empty channel / stencil count");
    const int code = kz * 100 + kx * 10 + ky;
    if (!conv_mfma_supported(code))
        return fail(APRNET_ERR_UNSUPPORTED, "conv_backward: bfloat16 features are supported for the 3x3x3, 1x3x3 and 1x5x5 stencils");
    const int64_t nt = p->tree_parts(d), np = p->number_parts(d);
    if ((gx && (!gx32_ws || ldgx32 < np)) || (nt > 0 && (!tree_ws || ldt < nt || (gx && (!gtree_ws || ldgt < nt)))))
        return fail(APRNET_ERR_INVALID_ARGUMENT, "conv_backward: work space too small");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    if (int rc = fill_tree_for_conv(p, d, x, ldx, Cin, tree_ws, ldt, st, nullptr)) return rc;
    if (gx) {
        fill2d<float>(gx32_ws, ldgx32, np, Cin, 0.f, st);
        fill2d<float>(gtree_ws, ldgt, nt, Cin, 0.f, st);
    }
    const bool flat = (kz == 1);
    TileList tl, near;
    if (int rc = get_tiles(p, d, flat ? 1 : 2, flat ? 8 : 4, &tl, st)) return rc;
    if (int rc = get_tiles(p, d, flat ? 1 : 2, flat ? 8 : 4, &near, st, 1)) return rc;
    if (tl.n > 0) {
        ConvArgs<bf16_t> a{};
        a.apr = p->dapr; a.tree = p->dtree; a.tiles = tl.d_tiles; a.n_tiles = tl.n;
        a.x = x; a.ldx = ldx; a.Cin = Cin; a.w = w; a.S_exp = S_exp; a.Cout = Cout;
        a.tree_data = tree_ws; a.ldt = ldt; a.Lc = p->lc(d); a.tree_off = p->tree_offset(a.Lc);
        a.x_count = np; a.t_count = nt;
        a.gy = gy; a.ldy = ldy; a.gx = gx32_ws; a.ldgx = ldgx32; a.gtree = gtree_ws; a.ldgt = ldgt; a.gw = gw;
        ConvArgs<bf16_t> b = a;
        b.tiles = near.d_tiles; b.n_tiles = near.n;
        b.x = gy; b.ldx = ldy; b.Cin = Cout; b.Cout = Cin; b.bias = nullptr;
        b.tree_data = nullptr; b.t_count = 0;
        // input gradient: bfloat16 products on the input-gradient lists of the plan when they are there, otherwise
        // (lists off or not buildable, fp32 products asked for) the scanning kernel with fp32 products
        if (!gx) near.n = 0;              // no input gradient asked for
        // weight gradient on the side stream, next to the input gradient
        if (int rc = set_conv_lists(p, d, code, tl, a, st)) return rc;
        // everything that can allocate or fail on the host comes before the fork
        if (near.n > 0 && bf16_math())
            if (int rc = set_conv_dx_lists(p, d, code, near, b, st)) return rc;
        const size_t wbytes = (conv_packed_bf16_bytes(code, S_exp, Cin, Cout) + 255) / 256 * 256;
        const size_t ng = (size_t)(Cout + 7) / 8, ibytes = ng * (size_t)np * 16;
        const bool regroup = bf16_regroup() && np < (1ll << 28) && ibytes <= ((size_t)32 << 30);
        size_t need = 0;
        if (near.n > 0) need = b.tile_win ? wbytes + (regroup ? ibytes : 0) : conv_packed_floats(code, S_exp, Cin, Cout, true) * sizeof(float);
        need = (need + 255) / 256 * 256;
        const size_t pbytes = bwd_deterministic() ? conv_dw_partial_bytes(code, Cout, Cin) : 0;
        ScratchLease lease;      // before the join guard below: its hand-over event is recorded after the join
        if (need + pbytes) if (int rc = lease.acquire(p, need + pbytes, st)) return rc;
        if (pbytes) set_dw_partials(p, need, code, a);
        hipStream_t side = st;
        if (near.n > 0) if (int rc = fork_side(p, st, &side)) return rc;
        SideJoin guard(p, st, side);
        if (int rc = launch_conv_dw_mfma(code, a, tl, p->apr.level_min, side)) return rc;
        if (near.n > 0 && b.tile_win) {
            // the output gradient regrouped as [Cout / 8][particles][8] behind the packed weights, as in the forward pass
            if (int rc = pack_conv_weights_bf16(code, w, S_exp, Cin, Cout, p->d_scratch, st, true)) return rc;
            if (regroup) {
                bf16_t* gyi = (bf16_t*)((char*)p->d_scratch + wbytes);
                if (int rc = interleave8_bf16(gy, ldy, nullptr, 0, Cout, Cout, np, gyi, st)) return rc;
                b.xi = gyi; b.ti = nullptr; b.xi_ld = np; b.ti_ld = 0;
            }
            b.w = (const float*)p->d_scratch;
            if (int rc = launch_conv_dx_mfma_bf16(code, b, near.n, st)) return rc;
        } else if (near.n > 0) {
            if (int rc = pack_conv_weights(code, w, S_exp, Cin, Cout, true, (float*)p->d_scratch, st)) return rc;
            b.w = (const float*)p->d_scratch;
            b.tile_win = nullptr;
            if (int rc = launch_conv_dx_mfma(code, b, near.n, st)) return rc;
        }
        if (int rc = guard.join()) return rc;
    }
    if (!gx) return 0;
    if (int rc = fill_tree_bwd_for_conv(p, d, gx32_ws, ldgx32, Cin, gtree_ws, ldgt, st)) return rc;
    if (np > 0) {
        dim3 grid((unsigned)std::min<int64_t>((np + 255) / 256, 4096), (unsigned)Cin);
        hipLaunchKernelGGL(round_to_bf16_kernel, grid, dim3(256), 0, st, gx32_ws, ldgx32, gx, ldgx, np);
        APRNET_LAUNCH_CHECK("round_to_bf16_kernel");
    }
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
int aprnet_conv_bwd_bf16(const aprnet_plan* p, int d, int kz, int kx, int ky, const uint16_t* x, int64_t ldx, int Cin,
                         const float* w, int S_exp, int Cout, const uint16_t* gy, int64_t ldy, uint16_t* gx, int64_t ldgx,
                         float* gw, uint16_t* tree_ws, int64_t ldt, float* gx32_ws, int64_t ldgx32, float* gtree_ws,
                         int64_t ldgt, void* st) {
    return conv_bwd_bf16(p, d, kz, kx, ky, (const bf16_t*)x, ldx, Cin, w, S_exp, Cout, (const bf16_t*)gy, ldy, (bf16_t*)gx, ldgx,
                         gw, (bf16_t*)tree_ws, ldt, gx32_ws, ldgx32, gtree_ws, ldgt, (hipStream_t)st);
}
int aprnet_conv_bwd_f32(const aprnet_plan* p, int d, int kz, int kx, int ky, const float* x, int64_t ldx, int Cin,
                        const float* w, int S_exp, int Cout, const float* gy, int64_t ldy, float* gx, int64_t ldgx,
                        float* gw, float* tree_ws, int64_t ldt, float* gtree_ws, int64_t ldgt, void* st) {
    return conv_bwd<float>(p, d, kz, kx, ky, x, ldx, Cin, w, S_exp, Cout, gy, ldy, gx, ldgx, gw, tree_ws, ldt, gtree_ws,
                           ldgt, (hipStream_t)st);
}
int aprnet_conv_bwd_f64(const aprnet_plan* p, int d, int kz, int kx, int ky, const double* x, int64_t ldx, int Cin,
                        const double* w, int S_exp, int Cout, const double* gy, int64_t ldy, double* gx, int64_t ldgx,
                        double* gw, double* tree_ws, int64_t ldt, double* gtree_ws, int64_t ldgt, void* st) {
    return conv_bwd<double>(p, d, kz, kx, ky, x, ldx, Cin, w, S_exp, Cout, gy, ldy, gx, ldgx, gw, tree_ws, ldt, gtree_ws,
                            ldgt, (hipStream_t)st);
}
}
