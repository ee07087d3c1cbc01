// Child-table operators: bottom-up tree fill (mean of children), max-pool with argmax, constant
// upsampling, and their backward passes.  All are HBM-bound gathers/scatters: one thread per
// (tree node, group of `cpt` channels), tree nodes of one level are contiguous, so every access is
// coalesced along the node index and the eight child slots are read from slot-major planes, once for
// the channels of the thread.  The slots are 32 bytes per node: against 8 x 4 bytes of fp32 data per node and channel
// they cost 1/cpt of the data traffic on top, so cpt is as large as the launch allows (channels_per_thread).
#include "common.hpp"

namespace aprnet {

constexpr int TB = 256;
constexpr int CPT_COARSE = 4;   // channels per workgroup of the coarse-level kernels
constexpr int NB = 4;           // channels of one batch: all loads of a batch are issued before its first store

// Channels per thread of a launch over n nodes: up to 16 (32 for 2-byte features), halved while fewer than 2^20
// threads would remain (the chip holds 2^19 threads at a time).
static int channels_per_thread(int64_t n, int C, size_t elem_bytes) {
    int cpt = elem_bytes <= 2 ? 32 : 16;
    while (cpt > NB && n * ((C + cpt - 1) / cpt) < ((int64_t)1 << 20)) cpt >>= 1;
    return cpt;
}

// Walks the channels [c_begin, c_end) of a thread in batches of NB with two buffers: the loads of batch b + 1 are
// issued BEFORE the stores of batch b, so that waiting for those loads (memory operations complete in issue order)
// does not wait for the stores, and a thread has up to two batches of loads in flight.  The empty asm statements only
// pin that order for the compiler, which otherwise sinks the loads of a channel below the stores of the one before.
#define APRNET_ORDER() __asm__ volatile("" ::: "memory")
template <int NBT, typename Buf, typename Load, typename Use>
__device__ __forceinline__ void channel_pipeline(int c_begin, int c_end, Load load, Use use) {
    Buf a, b;
    load(c_begin, a);
    APRNET_ORDER();
    for (int c = c_begin; c < c_end; c += 2 * NBT) {
        if (c + NBT < c_end) load(c + NBT, b);
        APRNET_ORDER();
        use(c, a);
        APRNET_ORDER();
        if (c + NBT >= c_end) break;
        if (c + 2 * NBT < c_end) load(c + 2 * NBT, a);
        APRNET_ORDER();
        use(c + NBT, b);
        APRNET_ORDER();
    }
}
// Kernels that mostly store need less in flight than kernels that mostly load: two channels per batch.
#ifndef APRNET_NBS
#define APRNET_NBS 2
#endif
constexpr int NBS = APRNET_NBS;
template <typename A, int NBT = NB> struct KidVals { A v[NBT][8]; };
template <typename T, int NBT = NB> struct RowVals { T v[NBT]; };

// The eight child slots of one tree node, decoded once per thread.  Every load that follows is unconditional (a
// missing child reads element 0 of the particle plane and its value is dropped): a load under a per-lane branch
// makes the compiler wait for memory inside the branch, which serialises the eight children of every channel.
struct Kids {
    int32_t off[8];                 // index among the particles (>= 0 in the table) or among the tree nodes (~v)
    uint32_t tree_mask, has_mask;   // bit s: child s is a tree node / exists
    __device__ __forceinline__ void read(const int32_t* __restrict__ children, int64_t n_tree, int64_t t) {
        int32_t v[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) v[s] = children[(int64_t)s * n_tree + t];
        tree_mask = has_mask = 0;
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const bool has = v[s] != NO_CHILD, tr = has && v[s] < 0;
            off[s] = has ? (tr ? ~v[s] : v[s]) : 0;
            has_mask |= (uint32_t)has << s;
            tree_mask |= (uint32_t)tr << s;
        }
    }
    __device__ __forceinline__ bool has(int s) const { return (has_mask >> s) & 1u; }
    __device__ __forceinline__ bool tree(int s) const { return (tree_mask >> s) & 1u; }
    __device__ __forceinline__ int count() const { return __popc(has_mask); }
    template <typename T> __device__ __forceinline__ T* ptr(int s, T* part, T* tnode) const { return (tree(s) ? tnode : part) + off[s]; }
};

// val[k][s] = value of child s in channel c + k, k < NBT (channels past c_end repeat the last one; the caller drops them)
template <typename T, int NBT = NB>
__device__ __forceinline__ void load_children(const Kids& kd, const T* part, int64_t ldp, const T* tnode, int64_t ldt,
                                              int c, int c_end, KidVals<typename Num<T>::acc, NBT>& val) {
#pragma unroll
    for (int k = 0; k < NBT; ++k) {
        const int cc = min(c + k, c_end - 1);
        const T* pb = part + (int64_t)cc * ldp;
        const T* tb = tnode + (int64_t)cc * ldt;
#pragma unroll
        for (int s = 0; s < 8; ++s) val.v[k][s] = Num<T>::ld(*kd.ptr(s, pb, tb));
    }
}

// Children 2y and 2y + 1 of one (z, x) row are neighbours in memory when both are particles (or both tree nodes)
// with consecutive indices: one 8-byte store for the two (element-aligned) instead of two 4-byte stores (4- and
// 16-byte pairs for bfloat16 and double).  Stores need no wait, so these branches cost nothing.
// (The pair goes out as ONE vector value: a struct of two elements is split into two stores again, each of which
// fills only every other element of the lines it touches.)
template <typename T> struct Pair { T v[2]; };
template <int BYTES> struct PairBits;
template <> struct PairBits<4> { typedef uint32_t type __attribute__((aligned(2))); };
template <> struct PairBits<8> { typedef uint32_t type __attribute__((ext_vector_type(2), aligned(4))); };
template <> struct PairBits<16> { typedef uint32_t type __attribute__((ext_vector_type(4), aligned(8))); };
template <typename T>
__device__ __forceinline__ void store_children(const Kids& kd, T* part, T* tnode, const T (&val)[8]) {
#pragma unroll
    for (int s = 0; s < 8; s += 2) {
        if (kd.has(s) && kd.has(s + 1) && kd.tree(s) == kd.tree(s + 1) && kd.off[s + 1] == kd.off[s] + 1) {
            typedef typename PairBits<2 * sizeof(T)>::type B;
            Pair<T> pv;
            pv.v[0] = val[s]; pv.v[1] = val[s + 1];
            *reinterpret_cast<B*>(kd.ptr(s, part, tnode)) = __builtin_bit_cast(B, pv);
        } else {
            if (kd.has(s)) *kd.ptr(s, part, tnode) = val[s];
            if (kd.has(s + 1)) *kd.ptr(s + 1, part, tnode) = val[s + 1];
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
                                          int tree_first, int c_begin, int cpt) {
    Kids kd;
    kd.read(children, n_tree, t);
    // 1/cnt is a power of two (cnt = product of 1-or-2 per dimension, helpers.hpp:133-153)
    typedef typename Num<T>::acc A;
    const A scale = (A)(1.0f / (float)max(kd.count(), 1));
    const int c_end = min(C, c_begin + cpt);
    // tree children: a window of the feature planes (parents directly under the features) or the tree planes
    const T* tn = tree_child_from_x ? x + tree_off : tree;
    const int64_t ldn = tree_child_from_x ? ldx : ldt;
    channel_pipeline<NB, KidVals<A>>(c_begin, c_end,
        [&](int c, KidVals<A>& val) { load_children<T>(kd, x, ldx, tn, ldn, c, c_end, val); },
        [&](int c, const KidVals<A>& val) {
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                if (c + k >= c_end) break;
                A sum = 0;
#pragma unroll
                for (int pass = 0; pass < 2; ++pass) {
                    const bool want_tree = (pass == 0) == (tree_first != 0);
#pragma unroll
                    for (int s = 0; s < 8; ++s)
                        if (kd.has(s) && want_tree == kd.tree(s)) sum += val.v[k][s];
                }
                tree[(int64_t)(c + k) * ldt + t] = Num<T>::st(sum * scale);
            }
        });
}

template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_level_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end,
                       const T* __restrict__ x, int64_t ldx, int C, T* __restrict__ tree, int64_t ldt,
                       int64_t tree_off, int tree_child_from_x, int tree_first, int cpt) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * TB + threadIdx.x;
    if (t < t_end) fill_node<T>(children, n_tree, t, x, ldx, C, tree, ldt, tree_off, tree_child_from_x, tree_first, blockIdx.y * cpt, cpt);
}

// the same for the listed nodes only (ascending indices of one level)
template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_list_kernel(const int32_t* __restrict__ children, int64_t n_tree, const int32_t* __restrict__ nodes, int64_t count,
                      const T* __restrict__ x, int64_t ldx, int C, T* __restrict__ tree, int64_t ldt,
                      int64_t tree_off, int tree_child_from_x, int tree_first, int cpt) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i < count) fill_node<T>(children, n_tree, nodes[i], x, ldx, C, tree, ldt, tree_off, tree_child_from_x, tree_first, blockIdx.y * cpt, cpt);
}

// The coarse levels of the tree hold a few nodes each: one launch walks them all, finest first, one workgroup per
// group of CPT_COARSE channels (a level's parents read only values of the same channels, so a workgroup barrier between
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
            fill_node<T>(children, n_tree, t, x, ldx, C, tree, ldt, 0, 0, 0, blockIdx.x * CPT_COARSE, CPT_COARSE);
        __syncthreads();
    }
}

// helpers.hpp:255-350, parent-driven: every child has exactly one parent, so no write conflicts.
template <typename T>
__device__ __forceinline__ void fill_node_bwd(const int32_t* children, int64_t n_tree, int64_t t, T* gx, int64_t ldx,
                                              int C, T* gtree, int64_t ldt, int64_t tree_off, int tree_child_in_x,
                                              int c_begin, int cpt) {
    Kids kd;
    kd.read(children, n_tree, t);
    typedef typename Num<T>::acc A;
    const A scale = (A)(1.0f / (float)max(kd.count(), 1));
    const int c_end = min(C, c_begin + cpt);
    T* tn = tree_child_in_x ? gx + tree_off : gtree;
    const int64_t ldn = tree_child_in_x ? ldx : ldt;
    struct Buf { A g[NBS]; KidVals<A, NBS> val; };
    channel_pipeline<NBS, Buf>(c_begin, c_end,
        [&](int c, Buf& b) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) b.g[k] = Num<T>::ld(gtree[(int64_t)min(c + k, c_end - 1) * ldt + t]);
            load_children<T, NBS>(kd, (const T*)gx, ldx, (const T*)tn, ldn, c, c_end, b.val);
        },
        [&](int c, const Buf& b) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) {
                if (c + k >= c_end) break;
                T out[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) out[s] = Num<T>::st(b.val.v[k][s] + b.g[k] * scale);
                store_children<T>(kd, gx + (int64_t)(c + k) * ldx, tn + (int64_t)(c + k) * ldn, out);
            }
        });
}

template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_bwd_level_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end,
                           T* gx, int64_t ldx, int C, T* gtree, int64_t ldt,
                           int64_t tree_off, int tree_child_in_x, int cpt) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * TB + threadIdx.x;
    if (t < t_end) fill_node_bwd<T>(children, n_tree, t, gx, ldx, C, gtree, ldt, tree_off, tree_child_in_x, blockIdx.y * cpt, cpt);
}

// the coarse levels in one launch, coarsest first (a parent's share must have arrived before it is handed down)
template <typename T>
__global__ void __launch_bounds__(TB)
fill_tree_bwd_coarse_kernel(const int32_t* __restrict__ children, int64_t n_tree, const CoarseLevels lv, T* gx, int64_t ldx,
                            int C, T* gtree, int64_t ldt) {
    for (int i = 0; i < lv.n; ++i) {
        for (int64_t t = lv.begin[i] + threadIdx.x; t < lv.end[i]; t += TB)
            fill_node_bwd<T>(children, n_tree, t, gx, ldx, C, gtree, ldt, 0, 0, blockIdx.x * CPT_COARSE, CPT_COARSE);
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
                   int64_t* __restrict__ arg, int64_t ldi, int64_t in_tree_off, int cpt) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_out) return;
    const int c_begin = blockIdx.y * cpt, c_end = min(C, c_begin + cpt);
    if (i < n_copy) {
        channel_pipeline<NB, RowVals<T>>(c_begin, c_end,
            [&](int c, RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k) r.v[k] = x[(int64_t)min(c + k, c_end - 1) * ldx + i];
            },
            [&](int c, const RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k)
                    if (c + k < c_end) { y[(int64_t)(c + k) * ldy + i] = r.v[k]; arg[(int64_t)(c + k) * ldi + i] = 0; }
            });
        return;
    }
    Kids kd;
    kd.read(children, n_tree, t_begin + (i - n_copy));
    typedef typename Num<T>::acc A;
    channel_pipeline<NB, KidVals<A>>(c_begin, c_end,
        [&](int c, KidVals<A>& val) { load_children<T>(kd, x, ldx, x + in_tree_off, ldx, c, c_end, val); },
        [&](int c, const KidVals<A>& val) {
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                if (c + k >= c_end) break;
                A best = (A)(-1e17f);               // initial value of the output, maxpool.hpp:51
                int64_t best_i = 0;
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    if (kd.has(s) && !kd.tree(s) && val.v[k][s] > best) { best = val.v[k][s]; best_i = kd.off[s]; }
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    if (kd.tree(s) && val.v[k][s] > best) { best = val.v[k][s]; best_i = (int64_t)kd.off[s] + in_tree_off; }
                y[(int64_t)(c + k) * ldy + i] = Num<T>::st(best);
                arg[(int64_t)(c + k) * ldi + i] = best_i;
            }
        });
}

// maxpool.hpp:170-230 without the zero-fill pass: every input position of level Lc has exactly one
// parent, which writes either its gradient (if it was the argmax) or zero.
template <typename T>
__global__ void __launch_bounds__(TB)
maxpool_bwd_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_out,
                   int64_t t_begin, const T* __restrict__ gy, int64_t ldy, int C, T* __restrict__ gx, int64_t ldx,
                   const int64_t* __restrict__ arg, int64_t ldi, int64_t in_tree_off, int cpt) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_out) return;
    const int c_begin = blockIdx.y * cpt, c_end = min(C, c_begin + cpt);
    if (i < n_copy) {
        channel_pipeline<NB, RowVals<T>>(c_begin, c_end,
            [&](int c, RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k) r.v[k] = gy[(int64_t)min(c + k, c_end - 1) * ldy + i];
            },
            [&](int c, const RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k)
                    if (c + k < c_end) { gx[(int64_t)(c + k) * ldx + i] = r.v[k]; }
            });
        return;
    }
    Kids kd;
    kd.read(children, n_tree, t_begin + (i - n_copy));
    struct Buf { T g[NBS]; int64_t m[NBS]; };
    channel_pipeline<NBS, Buf>(c_begin, c_end,
        [&](int c, Buf& b) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) {
                const int cc = min(c + k, c_end - 1);
                b.g[k] = gy[(int64_t)cc * ldy + i];
                b.m[k] = arg[(int64_t)cc * ldi + i];
            }
        },
        [&](int c, const Buf& b) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) {
                if (c + k >= c_end) break;
                T* gxc = gx + (int64_t)(c + k) * ldx;
                T out[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    const int64_t j = (int64_t)kd.off[s] + (kd.tree(s) ? in_tree_off : 0);
                    out[s] = (j == b.m[k]) ? b.g[k] : Num<T>::st(0);
                }
                store_children<T>(kd, gxc, gxc + in_tree_off, out);
            }
        });
}

// ---------------------------------------------------------------------------- upsample (constant)
// Backward of upsample.hpp:72-141 (upsample.hpp:199-232).  Gradient slot i < n_copy: copy.  Otherwise downsampled
// particle = tree node t of level Lc: the sum of its children's gradients, particles first, then tree nodes.
template <typename T>
__global__ void __launch_bounds__(TB)
upsample_bwd_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_in,
                    int64_t t_begin, const T* __restrict__ src, int64_t lds, int C, T* __restrict__ dst, int64_t ldd,
                    int64_t out_tree_off, int cpt) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_in) return;
    const int c_begin = blockIdx.y * cpt, c_end = min(C, c_begin + cpt);
    if (i < n_copy) {
        channel_pipeline<NB, RowVals<T>>(c_begin, c_end,
            [&](int c, RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k) r.v[k] = src[(int64_t)min(c + k, c_end - 1) * lds + i];
            },
            [&](int c, const RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k)
                    if (c + k < c_end) { dst[(int64_t)(c + k) * ldd + i] = r.v[k]; }
            });
        return;
    }
    Kids kd;
    kd.read(children, n_tree, t_begin + (i - n_copy));
    typedef typename Num<T>::acc A;
    channel_pipeline<NB, KidVals<A>>(c_begin, c_end,
        [&](int c, KidVals<A>& val) { load_children<T>(kd, src, lds, src + out_tree_off, lds, c, c_end, val); },
        [&](int c, const KidVals<A>& val) {
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                if (c + k >= c_end) break;
                A sum = 0;
#pragma unroll
                for (int s = 0; s < 8; ++s) if (kd.has(s) && !kd.tree(s)) sum += val.v[k][s];
#pragma unroll
                for (int s = 0; s < 8; ++s) if (kd.tree(s)) sum += val.v[k][s];
                dst[(int64_t)(c + k) * ldd + i] = Num<T>::st(sum);
            }
        });
}

// upsample.hpp:72-141.  Input slot i < n_copy: copy.  Otherwise downsampled particle = tree node t of level Lc: its
// value goes to every child (particle of level Lc + 1, or tree node of level Lc + 1).
// (A child-driven form -- one thread per 16 bytes of consecutive outputs, the source index from a parent table -- writes
// perfectly coalesced lines but was no faster: each parent value is then fetched by up to four XCDs.)
template <typename T>
__global__ void __launch_bounds__(TB)
upsample_fwd_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_in,
                    int64_t t_begin, const T* __restrict__ src, int64_t lds, int C, T* __restrict__ dst, int64_t ldd,
                    int64_t out_tree_off, int cpt) {
    const int64_t i = (int64_t)blockIdx.x * TB + threadIdx.x;
    if (i >= n_in) return;
    const int c_begin = blockIdx.y * cpt, c_end = min(C, c_begin + cpt);
    if (i < n_copy) {
        channel_pipeline<NB, RowVals<T>>(c_begin, c_end,
            [&](int c, RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k) r.v[k] = src[(int64_t)min(c + k, c_end - 1) * lds + i];
            },
            [&](int c, const RowVals<T>& r) {
#pragma unroll
                for (int k = 0; k < NB; ++k)
                    if (c + k < c_end) { dst[(int64_t)(c + k) * ldd + i] = r.v[k]; }
            });
        return;
    }
    Kids kd;
    kd.read(children, n_tree, t_begin + (i - n_copy));
    channel_pipeline<NBS, RowVals<T, NBS>>(c_begin, c_end,
        [&](int c, RowVals<T, NBS>& r) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) r.v[k] = src[(int64_t)min(c + k, c_end - 1) * lds + i];
        },
        [&](int c, const RowVals<T, NBS>& r) {
#pragma unroll
            for (int k = 0; k < NBS; ++k) {
                if (c + k >= c_end) break;
                T* d_ = dst + (int64_t)(c + k) * ldd;
                T out[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) out[s] = r.v[k];
                store_children<T>(kd, d_, d_ + out_tree_off, out);
            }
        });
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
    if (int rc = check_rows(ldx, p->number_parts(d), "fill_tree_mean", "input")) return rc;
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    const int l_coarse = coarse_levels_end(p, l_top);            // levels level_min .. l_coarse go in one launch
    for (int l = l_top; l > l_coarse; --l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b) continue;
        const int cpt = channels_per_thread(e - b, C, sizeof(T));
        dim3 grid((unsigned)((e - b + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
        const int from_x = (l + 1 == Lc);
        hipLaunchKernelGGL(fill_tree_level_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, b, e, x, ldx, C,
                           tree, ldt, from_x ? p->tree_offset(Lc) : 0, from_x, from_x, cpt);
    }
    CoarseLevels lv{};
    for (int l = l_coarse; l >= p->tree.level_min; --l)
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
    if (lv.n > 0)
        hipLaunchKernelGGL(fill_tree_coarse_kernel<T>, dim3((unsigned)((C + CPT_COARSE - 1) / CPT_COARSE)), dim3(TB), 0, st, p->d_children, p->n_tree,
                           lv, x, ldx, C, tree, ldt);
    APRNET_LAUNCH_CHECK("fill_tree kernels");
    return 0;
}

// fill_tree_mean for the nodes a convolution reads (`need`, see need.hip): the other nodes of the work space keep
// whatever they held.  Same arithmetic per node, so the values that are computed are those of the full fill.
template <typename T>
int fill_tree_mean_needed(const aprnet_plan* p, int d, const NeedLists& need, const T* x, int64_t ldx, int C, T* tree, int64_t ldt,
                          hipStream_t st) {
    if (C <= 0 || need.n_nodes == 0) return 0;
    const int Lc = p->lc(d);
    if (ldt < p->tree_parts(d)) return fail(APRNET_ERR_INVALID_ARGUMENT, "fill_tree_mean: tree work space too small");
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    const int l_coarse = coarse_levels_end(p, l_top);
    for (int l = l_top; l > l_coarse; --l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b || need.cnt[l] == 0) continue;
        const int from_x = (l + 1 == Lc);
        if (need.whole[l]) {
            const int cpt = channels_per_thread(e - b, C, sizeof(T));
            dim3 grid((unsigned)((e - b + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
            hipLaunchKernelGGL(fill_tree_level_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, b, e, x, ldx, C,
                               tree, ldt, from_x ? p->tree_offset(Lc) : 0, from_x, from_x, cpt);
        } else {
            const int cpt = channels_per_thread(need.cnt[l], C, sizeof(T));
            dim3 grid((unsigned)((need.cnt[l] + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
            hipLaunchKernelGGL(fill_tree_list_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, need.d_nodes + need.off[l],
                               need.cnt[l], x, ldx, C, tree, ldt, from_x ? p->tree_offset(Lc) : 0, from_x, from_x, cpt);
        }
    }
    CoarseLevels lv{};
    bool any = false;
    for (int l = l_coarse; l >= p->tree.level_min; --l) {
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
        any = any || need.cnt[l] > 0;
    }
    if (lv.n > 0 && any)          // the coarse levels (a few thousand nodes together) are filled whole, in one launch
        hipLaunchKernelGGL(fill_tree_coarse_kernel<T>, dim3((unsigned)((C + CPT_COARSE - 1) / CPT_COARSE)), dim3(TB), 0, st, p->d_children, p->n_tree,
                           lv, x, ldx, C, tree, ldt);
    APRNET_LAUNCH_CHECK("fill_tree kernels (needed nodes)");
    return 0;
}

template <typename T>
int fill_tree_mean_bwd(const aprnet_plan* p, int d, T* gx, int64_t ldx, int C, T* gtree, int64_t ldt, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "fill_tree_mean_bwd")) return rc;
    if (C <= 0) return 0;
    if (int rc = check_rows(ldx, p->number_parts(d), "fill_tree_mean_bwd", "input gradient")) return rc;
    if (int rc = check_rows(ldt, p->tree_parts(d), "fill_tree_mean_bwd", "tree gradient")) return rc;
    const int Lc = p->lc(d);
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    const int l_coarse = coarse_levels_end(p, l_top);
    CoarseLevels lv{};
    for (int l = p->tree.level_min; l <= l_coarse; ++l)
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
    if (lv.n > 0)
        hipLaunchKernelGGL(fill_tree_bwd_coarse_kernel<T>, dim3((unsigned)((C + CPT_COARSE - 1) / CPT_COARSE)), dim3(TB), 0, st, p->d_children,
                           p->n_tree, lv, gx, ldx, C, gtree, ldt);
    for (int l = std::max(l_coarse + 1, p->tree.level_min); l <= l_top; ++l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b) continue;
        const int cpt = channels_per_thread(e - b, C, sizeof(T));
        dim3 grid((unsigned)((e - b + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
        const int in_x = (l + 1 == Lc);
        hipLaunchKernelGGL(fill_tree_bwd_level_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, b, e, gx, ldx, C,
                           gtree, ldt, in_x ? p->tree_offset(Lc) : 0, in_x, cpt);
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
    if (int rc = check_rows(ldx, p->number_parts(d), "maxpool_forward", "input")) return rc;
    if (int rc = check_rows(ldy, n_out, "maxpool_forward", "output")) return rc;
    if (arg) if (int rc = check_rows(ldi, n_out, "maxpool_forward", "index output")) return rc;
    const int cpt = channels_per_thread(n_out, C, sizeof(T));
    dim3 grid((unsigned)((n_out + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
    hipLaunchKernelGGL(maxpool_fwd_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_out,
                       p->tree.level_begin(Lc - 1), x, ldx, C, y, ldy, arg, ldi, p->tree_offset(Lc), cpt);
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
    if (int rc = check_rows(ldx, p->number_parts(d), "maxpool_backward", "input gradient")) return rc;
    if (int rc = check_rows(ldy, n_out, "maxpool_backward", "output gradient")) return rc;
    if (int rc = check_rows(ldi, n_out, "maxpool_backward", "index input")) return rc;
    const int cpt = channels_per_thread(n_out, C, sizeof(T));
    dim3 grid((unsigned)((n_out + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
    hipLaunchKernelGGL(maxpool_bwd_kernel<T>, grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_out,
                       p->tree.level_begin(Lc - 1), gy, ldy, C, gx, ldx, arg, ldi, p->tree_offset(Lc), cpt);
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
    // forward: src at level delta d, dst at d - 1; backward: src is the gradient at d - 1, dst the gradient at d
    if (int rc = check_rows(lds, Backward ? p->number_parts(d - 1) : n_in, "upsample_const", Backward ? "output gradient" : "input")) return rc;
    if (int rc = check_rows(ldd, Backward ? n_in : p->number_parts(d - 1), "upsample_const", Backward ? "input gradient" : "output")) return rc;
    const int cpt = channels_per_thread(n_in, C, sizeof(T));
    dim3 grid((unsigned)((n_in + TB - 1) / TB), (unsigned)((C + cpt - 1) / cpt));
    hipLaunchKernelGGL((Backward ? upsample_bwd_kernel<T> : upsample_fwd_kernel<T>), grid, dim3(TB), 0, st, p->d_children, p->n_tree, n_copy, n_in,
                       p->tree.level_begin(Lc), src, lds, C, dst, ldd, p->tree_offset(Lc + 1), cpt);
    APRNET_LAUNCH_CHECK("upsample kernel");
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
// `need`: fill only the nodes the convolution's window lists read (null: every node)
int fill_tree_for_conv(const aprnet_plan* p, int d, const float* x, int64_t ldx, int C, float* tree, int64_t ldt, hipStream_t st,
                       const NeedLists* need) {
    return need ? fill_tree_mean_needed<float>(p, d, *need, x, ldx, C, tree, ldt, st) : fill_tree_mean<float>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_for_conv(const aprnet_plan* p, int d, const double* x, int64_t ldx, int C, double* tree, int64_t ldt, hipStream_t st,
                       const NeedLists* need) {
    return need ? fill_tree_mean_needed<double>(p, d, *need, x, ldx, C, tree, ldt, st) : fill_tree_mean<double>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_for_conv(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int C, bf16_t* tree, int64_t ldt, hipStream_t st,
                       const NeedLists* need) {
    return need ? fill_tree_mean_needed<bf16_t>(p, d, *need, x, ldx, C, tree, ldt, st) : fill_tree_mean<bf16_t>(p, d, x, ldx, C, tree, ldt, st);
}
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, float* gx, int64_t ldx, int C, float* gt, int64_t ldt, hipStream_t st) {
    return fill_tree_mean_bwd<float>(p, d, gx, ldx, C, gt, ldt, st);
}
int fill_tree_bwd_for_conv(const aprnet_plan* p, int d, double* gx, int64_t ldx, int C, double* gt, int64_t ldt, hipStream_t st) {
    return fill_tree_mean_bwd<double>(p, d, gx, ldx, C, gt, ldt, st);
}
}  // namespace aprnet
