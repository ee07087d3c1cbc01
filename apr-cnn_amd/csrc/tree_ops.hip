// Child-table operators: bottom-up tree fill (mean of children), max-pool with argmax, constant
// upsampling, and their backward passes.  All are HBM-bound gathers/scatters: one thread per
// (tree node, group of CPT channels), tree nodes of one level are contiguous, so every access is
// coalesced along the node index and the eight child slots are read from slot-major planes, once for
// the CPT channels of the thread (the index traffic would otherwise equal the data traffic).
#include "common.hpp"

namespace aprnet {

constexpr int TB = 256;
constexpr int CPT = 4;          // channels per thread

// Children 2y and 2y + 1 of one (z, x) row are neighbours in memory when both are particles (or both tree nodes)
// with consecutive indices: one 8-byte access for the two (element-aligned) instead of two 4-byte accesses whose
// lanes each use half of every 8 bytes (4- and 16-byte pairs for bfloat16 and double).
template <typename T> struct Pair { T v[2]; };        // alignment of one element

// val[s] = value of child s (0 where there is none); particles from `part`, tree nodes from `tnode[~v]`.
template <typename T>
__device__ __forceinline__ void load_children(const int32_t (&ch)[8], const T* part,
                                              const T* tnode, typename Num<T>::acc (&val)[8]) {
    typedef typename Num<T>::acc A;
#pragma unroll
    for (int s = 0; s < 8; s += 2) {
        const int32_t v0 = ch[s], v1 = ch[s + 1];
        bool paired = false;
        if constexpr (sizeof(T) >= 2) {
            const bool pp = v0 >= 0 && v1 == v0 + 1;
            const bool tt = v0 < 0 && v0 != NO_CHILD && v1 == v0 - 1;
            if (pp || tt) {
                const T* src = pp ? part + v0 : tnode + ~v0;
                const Pair<T> pv = *reinterpret_cast<const Pair<T>*>(src);
                val[s] = Num<T>::ld(pv.v[0]); val[s + 1] = Num<T>::ld(pv.v[1]);
                paired = true;
            }
        }
        if (!paired) {
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
                const int32_t v = k2 ? v1 : v0;
                A r = 0;
                if (v >= 0) r = Num<T>::ld(part[v]);
                else if (v != NO_CHILD) r = Num<T>::ld(tnode[~v]);
                val[s + k2] = r;
            }
        }
    }
}

// Writes val[s] to child s for every existing child, pairs in one 8-byte store.
template <typename T>
__device__ __forceinline__ void store_children(const int32_t (&ch)[8], T* part, T* tnode,
                                               const T (&val)[8]) {
#pragma unroll
    for (int s = 0; s < 8; s += 2) {
        const int32_t v0 = ch[s], v1 = ch[s + 1];
        bool paired = false;
        if constexpr (sizeof(T) >= 2) {
            const bool pp = v0 >= 0 && v1 == v0 + 1;
            const bool tt = v0 < 0 && v0 != NO_CHILD && v1 == v0 - 1;
            if (pp || tt) {
                Pair<T> pv;
                pv.v[0] = val[s]; pv.v[1] = val[s + 1];
                *reinterpret_cast<Pair<T>*>(pp ? part + v0 : tnode + ~v0) = pv;
                paired = true;
            }
        }
        if (!paired) {
#pragma unroll
            for (int k2 = 0; k2 < 2; ++k2) {
                const int32_t v = k2 ? v1 : v0;
                if (v >= 0) part[v] = val[s + k2];
                else if (v != NO_CHILD) tnode[~v] = val[s + k2];
            }
        }
    }
}

// ---------------------------------------------------------------------------- tree fill (mean)
// helpers.hpp:156-252.  One launch per tree level, finest first.  `tree_first`: the reference adds
// the downsampled particles before the particles for parents of level Lc-1 (pass order :174-224) and
// particles before tree nodes for coarser parents (:201-250); the same order is kept so the fp32
// sums agree to the last bit.
template <typename T>
__device__ __forceinline__ void fill_node(const int32_t* children, int64_t n_tree, int64_t t, const T* x, int64_t ldx,
                                          int C, T* tree, int64_t ldt, int64_t tree_off, int tree_child_from_x,
                                          int tree_first, int cg) {
    int32_t ch[8];
    int cnt = 0;
#pragma unroll
    for (int s = 0; s < 8; ++s) { ch[s] = children[(int64_t)s * n_tree + t]; cnt += ch[s] != NO_CHILD; }
    // 1/cnt is a power of two (cnt = product of 1-or-2 per dimension, helpers.hpp:133-153)
    typedef typename Num<T>::acc A;
    const A scale = (A)(1.0f / (float)max(cnt, 1));
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
        const int c = cg * CPT + k;
        if (c >= C) break;
        const T* xc = x + (int64_t)c * ldx;
        T* tc = tree + (int64_t)c * ldt;
        A val[8];
        load_children<T>(ch, xc, tree_child_from_x ? xc + tree_off : tc, val);
        A sum = 0;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const bool want_tree = (pass == 0) == (tree_first != 0);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const int32_t v = ch[s];
                if (v == NO_CHILD) continue;
                if (want_tree == (v < 0)) sum += val[s];
            }
        }
        tc[t] = Num<T>::st(sum * scale);
    }
}

template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_level_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end,
                       const T* __restrict__ x, int64_t ldx, int C, T* __restrict__ tree, int64_t ldt,
                       int64_t tree_off, int tree_child_from_x, int tree_first) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * TB + threadIdx.x;
    if (t < t_end) fill_node<T>(children, n_tree, t, x, ldx, C, tree, ldt, tree_off, tree_child_from_x, tree_first, blockIdx.y);
}

// The coarse levels of the tree hold a few nodes each: one launch walks them all, finest first, one workgroup per
// group of CPT channels (a level's parents read only values of the same channels, so a workgroup barrier between
// levels is enough).  Tree children come from the tree itself (none of these levels sits directly under the features),
// particle children from the feature vector as always.
constexpr int MAX_COARSE = 12;
struct CoarseLevels { int n; int64_t begin[MAX_COARSE], end[MAX_COARSE]; };
constexpr int64_t COARSE_NODES = 2048;      // levels are merged while they hold at most this many nodes together

template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_coarse_kernel(const int32_t* __restrict__ children, int64_t n_tree, const CoarseLevels lv, const T* x, int64_t ldx,
                        int C, T* tree, int64_t ldt) {
    for (int i = 0; i < lv.n; ++i) {
        for (int64_t t = lv.begin[i] + threadIdx.x; t < lv.end[i]; t += TB)
            fill_node<T>(children, n_tree, t, x, ldx, C, tree, ldt, 0, 0, 0, blockIdx.x);
        __syncthreads();
    }
}

// helpers.hpp:255-350, parent-driven: every child has exactly one parent, so no write conflicts.
template <typename T>
__device__ __forceinline__ void fill_node_bwd(const int32_t* children, int64_t n_tree, int64_t t, T* gx, int64_t ldx,
                                              int C, T* gtree, int64_t ldt, int64_t tree_off, int tree_child_in_x, int cg) {
    int32_t ch[8];
    int cnt = 0;
#pragma unroll
    for (int s = 0; s < 8; ++s) { ch[s] = children[(int64_t)s * n_tree + t]; cnt += ch[s] != NO_CHILD; }
    typedef typename Num<T>::acc A;
    const A scale = (A)(1.0f / (float)max(cnt, 1));
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
        const int c = cg * CPT + k;
        if (c >= C) break;
        T* gxc = gx + (int64_t)c * ldx;
        T* gtc = gtree + (int64_t)c * ldt;
        const A g = Num<T>::ld(gtc[t]) * scale;
        T* gt_child = tree_child_in_x ? gxc + tree_off : gtc;
        A val[8];
        load_children<T>(ch, gxc, gt_child, val);
        T out[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) out[s] = Num<T>::st(val[s] + g);
        store_children<T>(ch, gxc, gt_child, out);
    }
}

template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_bwd_level_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end,
                           T* __restrict__ gx, int64_t ldx, int C, T* __restrict__ gtree, int64_t ldt,
                           int64_t tree_off, int tree_child_in_x) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * TB + threadIdx.x;
    if (t < t_end) fill_node_bwd<T>(children, n_tree, t, gx, ldx, C, gtree, ldt, tree_off, tree_child_in_x, blockIdx.y);
}

// the coarse levels in one launch, coarsest first (a parent's share must have arrived before it is handed down)
template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_bwd_coarse_kernel(const int32_t* __restrict__ children, int64_t n_tree, const CoarseLevels lv, T* gx, int64_t ldx,
                            int C, T* gtree, int64_t ldt) {
    for (int i = 0; i < lv.n; ++i) {
        for (int64_t t = lv.begin[i] + threadIdx.x; t < lv.end[i]; t += TB)
            fill_node_bwd<T>(children, n_tree, t, gx, ldx, C, gtree, ldt, 0, 0, blockIdx.x);
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------- max pool
// maxpool.hpp:67-146.  Output slot i < n_copy: copy.  Otherwise parent node t of level Lc-1: first
// strict maximum over its children in the order (dz, dx, dy), particles before downsampled particles.
template <typename T>
__global__ void __launch_bounds__(TB)
maxpool_fwd_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_out,
                   int64_t t_begin, const T* __restrict__ x, int64_t ldx, int C, T* __restrict__ y, int64_t ldy,
                   int64_t* __restrict__ arg, int64_t ldi, int64_t in_tree_off) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_out) return;
    if (i < n_copy) {
#pragma unroll
        for (int k = 0; k < CPT; ++k) {
            const int c = blockIdx.y * CPT + k;
            if (c >= C) break;
            y[(int64_t)c * ldy + i] = x[(int64_t)c * ldx + i]; arg[(int64_t)c * ldi + i] = 0;
        }
        return;
    }
    const int64_t t = t_begin + (i - n_copy);
    int32_t ch[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) ch[s] = children[(int64_t)s * n_tree + t];
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
        const int c = blockIdx.y * CPT + k;
        if (c >= C) break;
        const T* xc = x + (int64_t)c * ldx;
        typedef typename Num<T>::acc A;
        A best = (A)(-1e17f);               // initial value of the output, maxpool.hpp:51
        int64_t best_i = 0;
        A val[8];
        load_children<T>(ch, xc, xc + in_tree_off, val);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int32_t v = ch[s];
            if (v >= 0 && val[s] > best) { best = val[s]; best_i = v; }
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int32_t v = ch[s];
            if (v < 0 && v != NO_CHILD && val[s] > best) { best = val[s]; best_i = (int64_t)(~v) + in_tree_off; }
        }
        y[(int64_t)c * ldy + i] = Num<T>::st(best);
        arg[(int64_t)c * ldi + i] = best_i;
    }
}

// maxpool.hpp:170-230 without the zero-fill pass: every input position of level Lc has exactly one
// parent, which writes either its gradient (if it was the argmax) or zero.
template <typename T>
__global__ void __launch_bounds__(TB)
maxpool_bwd_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_out,
                   int64_t t_begin, const T* __restrict__ gy, int64_t ldy, int C, T* __restrict__ gx, int64_t ldx,
                   const int64_t* __restrict__ arg, int64_t ldi, int64_t in_tree_off) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_out) return;
    if (i < n_copy) {
#pragma unroll
        for (int k = 0; k < CPT; ++k) {
            const int c = blockIdx.y * CPT + k;
            if (c >= C) break;
            gx[(int64_t)c * ldx + i] = gy[(int64_t)c * ldy + i];
        }
        return;
    }
    const int64_t t = t_begin + (i - n_copy);
    int32_t ch[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) ch[s] = children[(int64_t)s * n_tree + t];
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
        const int c = blockIdx.y * CPT + k;
        if (c >= C) break;
        T* gxc = gx + (int64_t)c * ldx;
        const T g = gy[(int64_t)c * ldy + i];
        const int64_t m = arg[(int64_t)c * ldi + i];
        T out[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int32_t v = ch[s];
            const int64_t j = v >= 0 ? (int64_t)v : (int64_t)(~v) + in_tree_off;
            out[s] = (j == m) ? g : Num<T>::st(0);
        }
        store_children<T>(ch, gxc, gxc + in_tree_off, out);
    }
}

// ---------------------------------------------------------------------------- upsample (constant)
// upsample.hpp:72-141.  Input slot i < n_copy: copy.  Otherwise downsampled particle = tree node t of
// level Lc: its value goes to every child (particle of level Lc+1, or tree node of level Lc+1).
template <typename T, bool Backward>
__global__ void __launch_bounds__(TB)
upsample_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_in,
                int64_t t_begin, const T* __restrict__ src, int64_t lds, int C, T* __restrict__ dst, int64_t ldd,
                int64_t out_tree_off) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_in) return;
    // forward: src = input at d, dst = output at d-1.  backward: src = grad_output, dst = grad_input.
    if (i < n_copy) {
#pragma unroll
        for (int k = 0; k < CPT; ++k) {
            const int c = blockIdx.y * CPT + k;
            if (c >= C) break;
            dst[(int64_t)c * ldd + i] = src[(int64_t)c * lds + i];
        }
        return;
    }
    const int64_t t = t_begin + (i - n_copy);
    int32_t ch[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) ch[s] = children[(int64_t)s * n_tree + t];
#pragma unroll
    for (int k = 0; k < CPT; ++k) {
        const int c = blockIdx.y * CPT + k;
        if (c >= C) break;
        const T* s_ = src + (int64_t)c * lds;
        T* d_ = dst + (int64_t)c * ldd;
        if (!Backward) {
            T out[8];
#pragma unroll
            for (int s = 0; s < 8; ++s) out[s] = s_[i];
            store_children<T>(ch, d_, d_ + out_tree_off, out);
        } else {
            typename Num<T>::acc sum = 0, val[8];      // particles first, then tree nodes (upsample.hpp:199-232)
            load_children<T>(ch, s_, s_ + out_tree_off, val);
#pragma unroll
            for (int s = 0; s < 8; ++s) if (ch[s] >= 0) sum += val[s];
#pragma unroll
            for (int s = 0; s < 8; ++s) if (ch[s] < 0 && ch[s] != NO_CHILD) sum += val[s];
            d_[i] = Num<T>::st(sum);
        }
    }
}

// ---------------------------------------------------------------------------- host launchers
// Highest level l <= l_top - 1 such that levels level_min .. l hold at most COARSE_NODES nodes together (and are
// at most MAX_COARSE levels); level_min - 1 when there is none.  The level directly under the features (l_top when
// it is Lc - 1) is never merged: its children are read from the feature vector.
static int coarse_levels_end(const aprnet_plan* p, int l_top) {
    int64_t nodes = 0;
    int l = p->tree.level_min - 1;
    while (l + 1 < l_top && l + 1 - p->tree.level_min < MAX_COARSE) {
        nodes += p->tree.level_end(l + 1) - p->tree.level_begin(l + 1);
        if (nodes > COARSE_NODES) break;
        ++l;
    }
    return l;
}

template <typename T>
int fill_tree_mean(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* tree, int64_t ldt, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "fill_tree_mean")) return rc;
    if (C <= 0) return 0;
    const int Lc = p->lc(d);
    if (ldt < p->tree_parts(d)) return fail(APRNET_ERR_INVALID_ARGUMENT, "fill_tree_mean: tree work space too small");
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    const int l_coarse = coarse_levels_end(p, l_top);            // levels level_min .. l_coarse go in one launch
    for (int l = l_top; l > l_coarse; --l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b) continue;
        dim3 grid((unsigned)((e - b + TB - 1) / TB), (unsigned)((C + CPT - 1) / CPT));
        const int from_x = (l + 1 == Lc);
        hipLaunchKernelGGL(fill_tree_level_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, b, e, x, ldx, C,
                           tree, ldt, from_x ? p->tree_offset(Lc) : 0, from_x, from_x);
    }
    CoarseLevels lv{};
    for (int l = l_coarse; l >= p->tree.level_min; --l)
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
    if (lv.n > 0)
        hipLaunchKernelGGL(fill_tree_coarse_kernel<T>, dim3((unsigned)((C + CPT - 1) / CPT)), dim3(TB), 0, st, p->d_children, p->n_tree,
                           lv, x, ldx, C, tree, ldt);
    APRNET_LAUNCH_CHECK("fill_tree kernels");
    return 0;
}

template <typename T>
int fill_tree_mean_bwd(const aprnet_plan* p, int d, T* gx, int64_t ldx, int C, T* gtree, int64_t ldt, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "fill_tree_mean_bwd")) return rc;
    if (C <= 0) return 0;
    const int Lc = p->lc(d);
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    const int l_coarse = coarse_levels_end(p, l_top);
    CoarseLevels lv{};
    for (int l = p->tree.level_min; l <= l_coarse; ++l)
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
    if (lv.n > 0)
        hipLaunchKernelGGL(fill_tree_bwd_coarse_kernel<T>, dim3((unsigned)((C + CPT - 1) / CPT)), dim3(TB), 0, st, p->d_children,
                           p->n_tree, lv, gx, ldx, C, gtree, ldt);
    for (int l = std::max(l_coarse + 1, p->tree.level_min); l <= l_top; ++l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b) continue;
        dim3 grid((unsigned)((e - b + TB - 1) / TB), (unsigned)((C + CPT - 1) / CPT));
        const int in_x = (l + 1 == Lc);
        hipLaunchKernelGGL(fill_tree_bwd_level_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, b, e, gx, ldx, C,
                           gtree, ldt, in_x ? p->tree_offset(Lc) : 0, in_x);
    }
    APRNET_LAUNCH_CHECK("fill_tree_bwd_level_kernel");
    return 0;
}

template <typename T>
int maxpool_fwd(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* y, int64_t ldy, int64_t* arg,
                int64_t ldi, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "maxpool_forward")) return rc;
    const int Lc = p->lc(d);
    if (Lc - 1 < p->tree.level_min) return fail(APRNET_ERR_LEVEL_DELTA, "maxpool_forward: nothing left to pool");
    const int64_t n_out = p->number_parts(d + 1), n_copy = p->apr.level_end(Lc - 1);
    if (C <= 0 || n_out <= 0) return 0;
    dim3 grid((unsigned)((n_out + TB - 1) / TB), (unsigned)((C + CPT - 1) / CPT));
    hipLaunchKernelGGL(maxpool_fwd_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_out,
                       p->tree.level_begin(Lc - 1), x, ldx, C, y, ldy, arg, ldi, p->tree_offset(Lc));
    APRNET_LAUNCH_CHECK("maxpool_fwd_kernel");
    return 0;
}

template <typename T>
int maxpool_bwd(const aprnet_plan* p, int d, const T* gy, int64_t ldy, int C, T* gx, int64_t ldx, const int64_t* arg,
                int64_t ldi, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "maxpool_backward")) return rc;
    const int Lc = p->lc(d);
    if (Lc - 1 < p->tree.level_min) return fail(APRNET_ERR_LEVEL_DELTA, "maxpool_backward: invalid level delta");
    const int64_t n_out = p->number_parts(d + 1), n_copy = p->apr.level_end(Lc - 1);
    if (C <= 0 || n_out <= 0) return 0;
    dim3 grid((unsigned)((n_out + TB - 1) / TB), (unsigned)((C + CPT - 1) / CPT));
    hipLaunchKernelGGL(maxpool_bwd_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_out,
                       p->tree.level_begin(Lc - 1), gy, ldy, C, gx, ldx, arg, ldi, p->tree_offset(Lc));
    APRNET_LAUNCH_CHECK("maxpool_bwd_kernel");
    return 0;
}

template <typename T, bool Backward>
int upsample(const aprnet_plan* p, int d, const T* src, int64_t lds, int C, T* dst, int64_t ldd, hipStream_t st) {
    if (d <= 0)   // upsample.hpp:49-54
        return fail(APRNET_ERR_INVALID_ARGUMENT, "UpSampleConst is only implemented for downsampled particles: "
                                                 "input must have level_delta > 0");
    if (int rc = check_level_delta(p, d, "upsample_const")) return rc;
    const int Lc = p->lc(d);
    const int64_t n_in = p->number_parts(d), n_copy = p->apr.level_end(Lc);
    if (C <= 0 || n_in <= 0) return 0;
    dim3 grid((unsigned)((n_in + TB - 1) / TB), (unsigned)((C + CPT - 1) / CPT));
    hipLaunchKernelGGL((upsample_kernel<T, Backward>), grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_in,
                       p->tree.level_begin(Lc), src, lds, C, dst, ldd, p->tree_offset(Lc + 1));
    APRNET_LAUNCH_CHECK("upsample_kernel");
    return 0;
}

}  // namespace aprnet

using namespace aprnet;

extern "C" {

#define TREE_OPS_API(T, SFX)                                                                                          \
    int aprnet_fill_tree_mean_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* tree, int64_t ldt, \
                                    void* st) { return fill_tree_mean<T>(p, d, x, ldx, C, tree, ldt, (hipStream_t)st); } \
    int aprnet_fill_tree_mean_bwd_##SFX(const aprnet_plan* p, int d, T* gx, int64_t ldx, int C, T* gt, int64_t ldt,    \
                                        void* st) { return fill_tree_mean_bwd<T>(p, d, gx, ldx, C, gt, ldt, (hipStream_t)st); } \
    int aprnet_maxpool_fwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* y, int64_t ldy,       \
                                 int64_t* arg, int64_t ldi, void* st) {                                                \
        return maxpool_fwd<T>(p, d, x, ldx, C, y, ldy, arg, ldi, (hipStream_t)st); }                                   \
    int aprnet_maxpool_bwd_##SFX(const aprnet_plan* p, int d, const T* gy, int64_t ldy, int C, T* gx, int64_t ldx,     \
                                 const int64_t* arg, int64_t ldi, void* st) {                                          \
        return maxpool_bwd<T>(p, d, gy, ldy, C, gx, ldx, arg, ldi, (hipStream_t)st); }                                 \
    int aprnet_upsample_fwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* y, int64_t ldy,      \
                                  void* st) { return upsample<T, false>(p, d, x, ldx, C, y, ldy, (hipStream_t)st); }   \
    int aprnet_upsample_bwd_##SFX(const aprnet_plan* p, int d, const T* gy, int64_t ldy, int C, T* gx, int64_t ldx,    \
                                  void* st) { return upsample<T, true>(p, d, gy, ldy, C, gx, ldx, (hipStream_t)st); }

TREE_OPS_API(float, f32)
TREE_OPS_API(double, f64)
// bfloat16 storage (uint16_t bit patterns at the boundary), fp32 arithmetic
#define TREE_OPS_BF16(NAME, ARGS, CALL)                                                                              \
    int aprnet_##NAME##_bf16 ARGS { typedef bf16_t B; return CALL; }
TREE_OPS_BF16(fill_tree_mean, (const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* tree, int64_t ldt, void* st),
              fill_tree_mean<B>(p, d, (const B*)x, ldx, C, (B*)tree, ldt, (hipStream_t)st))
TREE_OPS_BF16(fill_tree_mean_bwd, (const aprnet_plan* p, int d, uint16_t* gx, int64_t ldx, int C, uint16_t* gt, int64_t ldt, void* st),
              fill_tree_mean_bwd<B>(p, d, (B*)gx, ldx, C, (B*)gt, ldt, (hipStream_t)st))
TREE_OPS_BF16(maxpool_fwd, (const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy, int64_t* arg, int64_t ldi, void* st),
              maxpool_fwd<B>(p, d, (const B*)x, ldx, C, (B*)y, ldy, arg, ldi, (hipStream_t)st))
TREE_OPS_BF16(maxpool_bwd, (const aprnet_plan* p, int d, const uint16_t* gy, int64_t ldy, int C, uint16_t* gx, int64_t ldx, const int64_t* arg, int64_t ldi, void* st),
              maxpool_bwd<B>(p, d, (const B*)gy, ldy, C, (B*)gx, ldx, arg, ldi, (hipStream_t)st))
TREE_OPS_BF16(upsample_fwd, (const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy, void* st),
              (upsample<B, false>(p, d, (const B*)x, ldx, C, (B*)y, ldy, (hipStream_t)st)))
TREE_OPS_BF16(upsample_bwd, (const aprnet_plan* p, int d, const uint16_t* gy, int64_t ldy, int C, uint16_t* gx, int64_t ldx, void* st),
              (upsample<B, true>(p, d, (const B*)gy, ldy, C, (B*)gx, ldx, (hipStream_t)st)))

}  // extern "C"

namespace aprnet {
// used by the convolution launchers (conv.hip, conv_bwd.hip)
int fill_tree_for_conv(const aprnet_plan* p, int d, const float* x, int64_t ldx, int C, float* tree, int64_t ldt, hipStream_t st) {
    return fill_tree_mean<float>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_for_conv(const aprnet_plan* p, int d, const double* x, int64_t ldx, int C, double* tree, int64_t ldt, hipStream_t st) {
    return fill_tree_mean<double>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_for_conv(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int C, bf16_t* tree, int64_t ldt, hipStream_t st) {
    return fill_tree_mean<bf16_t>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, float* gx, int64_t ldx, int C, float* gt, int64_t ldt, hipStream_t st) {
    return fill_tree_mean_bwd<float>(p, d, gx, ldx, C, gt, ldt, st);
}
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, double* gx, int64_t ldx, int C, double* gt, int64_t ldt, hipStream_t st) {
    return fill_tree_mean_bwd<double>(p, d, gx, ldx, C, gt, ldt, st);
}
}  // namespace aprnet
