// bfloat16 features grouped by eight channels: [C / 8][ld][8], the eight channels of a particle in one 16-byte word.
//
// The reference keeps channel planes [C][N] (conv.hpp:68).  On planes every operator of this library gathers one
// 2-byte value per channel and particle; grouped, a particle's eight channels come with one 16-byte access, which
// is what the bfloat16 convolution stages from anyway.  A network whose layers hand each other grouped tensors
// converts at its two ends only (regroup / ungroup below) and needs neither the per-call regrouping pass of the
// convolution nor two-byte stores in its epilogue.  The operators here are those of a network's forward pass:
// tree fill (for the convolution), max pool (values only: the argmax serves the backward pass), constant
// upsampling and the 1x1x1 convolution.  Arithmetic and summation order are those of the plane kernels
// (tree_ops.hip, conv111.hip), so results are bit-identical to theirs.
#include "common.hpp"

namespace aprnet {

constexpr int GTB = 256;

__device__ __forceinline__ void unpack8(const uint4 v, float (&f)[8]) {
    const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        f[2 * k] = __builtin_bit_cast(float, w[k] << 16);
        f[2 * k + 1] = __builtin_bit_cast(float, w[k] & 0xffff0000u);
    }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    unsigned w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k] = (unsigned)float_to_bf16(f[2 * k]).bits | ((unsigned)float_to_bf16(f[2 * k + 1]).bits << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}
__device__ __forceinline__ const uint4* g8_at(const bf16_t* base, int64_t ld, int q, int64_t i) {
    return reinterpret_cast<const uint4*>(base) + (int64_t)q * ld + i;
}
__device__ __forceinline__ uint4* g8_at(bf16_t* base, int64_t ld, int q, int64_t i) {
    return reinterpret_cast<uint4*>(base) + (int64_t)q * ld + i;
}

// ---------------------------------------------------------------------------- planes <-> groups
// out[q][i][c] = x[8 q + c][i]; channels past C read as zeros
__global__ void regroup8_kernel(const bf16_t* __restrict__ x, int64_t ldx, int C, int64_t n, bf16_t* __restrict__ out, int64_t ldo) {
    const int q = blockIdx.y;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        unsigned v[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] = (8 * q + c < C) ? x[(int64_t)(8 * q + c) * ldx + i].bits : 0u;
        *g8_at(out, ldo, q, i) = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
    }
}
__global__ void ungroup8_kernel(const bf16_t* __restrict__ xg, int64_t ldg, int C, int64_t n, bf16_t* __restrict__ out, int64_t ldo) {
    const int q = blockIdx.y;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        const uint4 v = *g8_at(xg, ldg, q, i);
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (8 * q + c < C) out[(int64_t)(8 * q + c) * ldo + i].bits = (unsigned short)(c & 1 ? w[c >> 1] >> 16 : w[c >> 1] & 0xffffu);
    }
}

// ---------------------------------------------------------------------------- tree fill (mean of children)
// fill_node of tree_ops.hip for eight channels at once: same pass order (downsampled particles before particles
// under the features, particles before tree nodes elsewhere), same fp32 sums.
__device__ __forceinline__ void fill_node_g8(const int32_t* children, int64_t n_tree, int64_t t, const bf16_t* x, int64_t ldx,
                                             bf16_t* tree, int64_t ldt, int64_t tree_off, int tree_child_from_x, int tree_first, int q) {
    int32_t ch[8];
    int cnt = 0;
#pragma unroll
    for (int s = 0; s < 8; ++s) { ch[s] = children[(int64_t)s * n_tree + t]; cnt += ch[s] != NO_CHILD; }
    const float scale = 1.0f / (float)max(cnt, 1);
    // unconditional loads (a missing child reads particle 0 and is skipped below): a load under a per-lane branch
    // makes the compiler wait for memory inside the branch, one child after the other
    uint4 raw[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int32_t v = ch[s];
        const bool from_tree = v < 0 && v != NO_CHILD && !tree_child_from_x;
        const int64_t idx = v >= 0 ? (int64_t)v : (v == NO_CHILD ? 0 : (tree_child_from_x ? tree_off + ~v : (int64_t)~v));
        raw[s] = *g8_at(from_tree ? (const bf16_t*)tree : x, from_tree ? ldt : ldx, q, idx);
    }
    float sum[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const bool want_tree = (pass == 0) == (tree_first != 0);
#pragma unroll
        for (int s = 0; s < 8; ++s) {
            const int32_t v = ch[s];
            if (v == NO_CHILD || want_tree != (v < 0)) continue;
            float f[8];
            unpack8(raw[s], f);
#pragma unroll
            for (int c = 0; c < 8; ++c) sum[c] += f[c];
        }
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) sum[c] *= scale;
    *g8_at(tree, ldt, q, t) = pack8(sum);
}

__global__ void __launch_bounds__(GTB)
fill_tree_level_g8_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end, const bf16_t* __restrict__ x,
                          int64_t ldx, bf16_t* __restrict__ tree, int64_t ldt, int64_t tree_off, int from_x, int tree_first, int G) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * GTB + threadIdx.x;
    if (t >= t_end) return;
    for (int q = 0; q < G; ++q) fill_node_g8(children, n_tree, t, x, ldx, tree, ldt, tree_off, from_x, tree_first, q);
}

__global__ void __launch_bounds__(GTB)
fill_tree_list_g8_kernel(const int32_t* __restrict__ children, int64_t n_tree, const int32_t* __restrict__ nodes, int64_t count,
                         const bf16_t* __restrict__ x, int64_t ldx, bf16_t* __restrict__ tree, int64_t ldt, int64_t tree_off, int from_x,
                         int tree_first, int G) {
    const int64_t i = (int64_t)blockIdx.x * GTB + threadIdx.x;
    if (i >= count) return;
    const int64_t t = nodes[i];
    // every channel group of the node in one thread: the list entry and the child table are read once
    for (int q = 0; q < G; ++q) fill_node_g8(children, n_tree, t, x, ldx, tree, ldt, tree_off, from_x, tree_first, q);
}

constexpr int G_MAX_COARSE = 12;
struct GCoarse { int n; int64_t begin[G_MAX_COARSE], end[G_MAX_COARSE]; };

// the coarse levels in one launch, finest first, one workgroup per channel group (see fill_tree_coarse_kernel)
__global__ void __launch_bounds__(GTB)
fill_tree_coarse_g8_kernel(const int32_t* __restrict__ children, int64_t n_tree, const GCoarse lv, const bf16_t* x, int64_t ldx,
                           bf16_t* tree, int64_t ldt) {
    for (int i = 0; i < lv.n; ++i) {
        for (int64_t t = lv.begin[i] + threadIdx.x; t < lv.end[i]; t += GTB)
            fill_node_g8(children, n_tree, t, x, ldx, tree, ldt, 0, 0, 0, blockIdx.x);
        __syncthreads();
    }
}

// need: fill only the nodes a convolution reads (see need.hip); null: every node
// particles_first: the level under the features sums its particles before its downsampled particles, as every other
// level sums particles before tree nodes (for the tree of an upsampled tensor, see tree_of_upsampled_g8)
int fill_tree_mean_g8(const aprnet_plan* p, int d, const bf16_t* x, int64_t ldx, int C, bf16_t* tree, int64_t ldt, hipStream_t st,
                      const NeedLists* need, bool particles_first) {
    if (C <= 0 || (need && need->n_nodes == 0)) return 0;
    if (C % 8) return fail(APRNET_ERR_INVALID_ARGUMENT, "grouped features hold a multiple of eight channels");
    const int Lc = p->lc(d), G = C / 8;
    if (ldt < p->tree_parts(d)) return fail(APRNET_ERR_INVALID_ARGUMENT, "fill_tree_mean: tree work space too small");
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    // levels level_min .. l_coarse (at most 2048 nodes together, never the level under the features) go in one launch
    int64_t nodes = 0;
    int l_coarse = p->tree.level_min - 1;
    while (l_coarse + 1 < l_top && l_coarse + 1 - p->tree.level_min < G_MAX_COARSE) {
        nodes += p->tree.level_end(l_coarse + 1) - p->tree.level_begin(l_coarse + 1);
        if (nodes > 2048) break;
        ++l_coarse;
    }
    for (int l = l_top; l > l_coarse; --l) {
        const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
        if (e <= b) continue;
        const int from_x = (l + 1 == Lc);
        if (need && need->cnt[l] == 0) continue;
        if (need && !need->whole[l])
            hipLaunchKernelGGL(fill_tree_list_g8_kernel, dim3((unsigned)((need->cnt[l] + GTB - 1) / GTB)), dim3(GTB), 0, st,
                               p->d_children, p->n_tree, need->d_nodes + need->off[l], need->cnt[l], x, ldx, tree, ldt,
                               from_x ? p->tree_offset(Lc) : 0, from_x, from_x && !particles_first, G);
        else
            hipLaunchKernelGGL(fill_tree_level_g8_kernel, dim3((unsigned)((e - b + GTB - 1) / GTB)), dim3(GTB), 0, st, p->d_children,
                               p->n_tree, b, e, x, ldx, tree, ldt, from_x ? p->tree_offset(Lc) : 0, from_x, from_x && !particles_first, G);
    }
    GCoarse lv{};
    for (int l = l_coarse; l >= p->tree.level_min; --l)
        if (p->tree.level_end(l) > p->tree.level_begin(l)) { lv.begin[lv.n] = p->tree.level_begin(l); lv.end[lv.n] = p->tree.level_end(l); ++lv.n; }
    if (lv.n > 0)
        hipLaunchKernelGGL(fill_tree_coarse_g8_kernel, dim3((unsigned)G), dim3(GTB), 0, st, p->d_children, p->n_tree, lv, x, ldx, tree, ldt);
    APRNET_LAUNCH_CHECK("fill_tree g8 kernels");
    return 0;
}

// The mean tree of u = UpSampleConst(z) without reading u.  z lives at level delta d + 1: particles up to level Lc - 1,
// then the nodes of level Lc - 1 in tree order ("downsampled particles").  The upsample gives all children of such a
// node the node's value, so the node's mean in the tree of u is that value again (a sum of k <= 8 equal bfloat16
// values and its division by k are exact in fp32), and below level Lc - 1 the tree of u is the tree of z.
__global__ void __launch_bounds__(GTB)
tree_level_from_coarse_g8_kernel(const int32_t* __restrict__ nodes, int64_t count, int64_t t_begin, int64_t n_copy,
                                 const bf16_t* __restrict__ z, int64_t ldz, bf16_t* __restrict__ tree, int64_t ldt) {
    const int64_t i = (int64_t)blockIdx.x * GTB + threadIdx.x;
    if (i >= count) return;
    const int64_t t = nodes ? (int64_t)nodes[i] : t_begin + i;
    *g8_at(tree, ldt, blockIdx.y, t) = *g8_at(z, ldz, blockIdx.y, n_copy + (t - t_begin));
}
int tree_of_upsampled_g8(const aprnet_plan* p, int d, const bf16_t* z, int64_t ldz, int C, bf16_t* tree, int64_t ldt, hipStream_t st,
                         const NeedLists* need) {
    if (C <= 0 || (need && need->n_nodes == 0)) return 0;
    if (C % 8) return fail(APRNET_ERR_INVALID_ARGUMENT, "grouped features hold a multiple of eight channels");
    if (int rc = check_level_delta(p, d + 1, "conv_forward (x2_coarse)")) return rc;
    if (int rc = check_rows(ldz, p->number_parts(d + 1), "conv_forward", "x2_coarse")) return rc;
    const int Lc = p->lc(d), l = Lc - 1;
    if (l > p->tree.level_max) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv_forward: x2_coarse needs a level below the features");
    // levels below Lc - 1: the tree of z (the lists of needed nodes name absolute levels, so they serve this fill too)
    // (in the tree of u the nodes of level Lc - 1 are tree nodes, summed after the particles of their level)
    if (int rc = fill_tree_mean_g8(p, d + 1, z, ldz, C, tree, ldt, st, need, true)) return rc;
    const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
    if (e <= b || (need && need->cnt[l] == 0)) return 0;
    const bool listed = need && !need->whole[l];
    const int64_t count = listed ? need->cnt[l] : e - b;
    hipLaunchKernelGGL(tree_level_from_coarse_g8_kernel, dim3((unsigned)((count + GTB - 1) / GTB), (unsigned)(C / 8)), dim3(GTB), 0, st,
                       listed ? need->d_nodes + need->off[l] : nullptr, count, b, p->apr.level_end(l), z, ldz, tree, ldt);
    APRNET_LAUNCH_CHECK("tree_level_from_coarse_g8_kernel");
    return 0;
}

// ---------------------------------------------------------------------------- max pool (values), upsample
// maxpool_fwd_kernel of tree_ops.hip without the argmax plane: candidate order (dz, dx, dy), particles before
// downsampled particles, strict >, start value -1e17 (maxpool.hpp:51, 88-143).
__global__ void __launch_bounds__(GTB)
maxpool_g8_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_out, int64_t t_begin,
                  const bf16_t* __restrict__ x, int64_t ldx, int G, bf16_t* __restrict__ y, int64_t ldy, int64_t in_tree_off) {
    const int64_t i = (int64_t)blockIdx.x * GTB + threadIdx.x;
    if (i >= n_out) return;
    if (i < n_copy) {
        for (int q = 0; q < G; ++q) *g8_at(y, ldy, q, i) = *g8_at(x, ldx, q, i);
        return;
    }
    const int64_t t = t_begin + (i - n_copy);
    int32_t ch[8];                        // read once for all channel groups
#pragma unroll
    for (int s = 0; s < 8; ++s) ch[s] = children[(int64_t)s * n_tree + t];
    for (int q = 0; q < G; ++q) {
        uint4 raw[8];                     // unconditional loads, as in fill_node_g8
#pragma unroll
        for (int s = 0; s < 8; ++s)
            raw[s] = *g8_at(x, ldx, q, ch[s] >= 0 ? (int64_t)ch[s] : (ch[s] == NO_CHILD ? 0 : in_tree_off + ~ch[s]));
        float best[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) best[c] = -1e17f;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass)
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                if (ch[s] == NO_CHILD || (pass == 0) != (ch[s] >= 0)) continue;
                float f[8];
                unpack8(raw[s], f);
#pragma unroll
                for (int c = 0; c < 8; ++c) if (f[c] > best[c]) best[c] = f[c];
            }
        *g8_at(y, ldy, q, i) = pack8(best);
    }
}

// upsample_fwd_kernel of tree_ops.hip: a downsampled particle's value goes to each of its children.  TWO lanes per
// parent, one for the children with even y and one for those with odd y: children 2y and 2y + 1 of a row are neighbours
// in memory, so the lanes of a wave write whole lines (one lane per parent would fill every other 16 bytes of them).
__global__ void __launch_bounds__(GTB)
upsample_g8_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t n_copy, int64_t n_in, int64_t t_begin,
                   const bf16_t* __restrict__ src, int64_t lds, int G, bf16_t* __restrict__ dst, int64_t ldd, int64_t out_tree_off) {
    const int64_t j = (int64_t)blockIdx.x * GTB + threadIdx.x;
    const int64_t n_par = n_in - n_copy;
    if (j < n_copy) {                     // copied positions: one lane each
        for (int q = 0; q < G; ++q) *g8_at(dst, ldd, q, j) = *g8_at(src, lds, q, j);
        return;
    }
    const int64_t k = j - n_copy;
    if (k >= 2 * n_par) return;
    const int64_t i = n_copy + (k >> 1), t = t_begin + (k >> 1);
    const int dy = (int)(k & 1);
    int64_t at[4];                        // the four children with this dy (slot = 2 * (2 dz + dx) + dy); -1: none
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int32_t c = children[(int64_t)(2 * p + dy) * n_tree + t];
        at[p] = c >= 0 ? (int64_t)c : (c != NO_CHILD ? out_tree_off + ~c : -1);
    }
    for (int q = 0; q < G; ++q) {
        const uint4 v = *g8_at(src, lds, q, i);
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (at[p] >= 0) *g8_at(dst, ldd, q, at[p]) = v;
    }
}

// ---------------------------------------------------------------------------- 1x1x1 convolution
// out[co][i] = bias[co] + sum_ci w[s][co][ci] x[ci][i], s constant over a range of particles (conv.hpp:199-256).
// One thread per (particle, group of eight outputs): the input groups come with 16-byte loads, the 8 x Cin weights of
// the output group sit in LDS and are read as broadcasts.  Bound by memory for the layers it serves (channel
// reductions of the decoder, the head).  OUT_G8: grouped output, otherwise channel planes (the head of a network).
constexpr int C111_MAX_CIN = 256;
constexpr int C111_OG = 4;        // output groups (of eight channels) per thread: the input is read once per 32 outputs

template <bool OUT_G8>
__global__ void __launch_bounds__(GTB)
conv111_g8_kernel(const bf16_t* __restrict__ x, int64_t ldx, int Cin, const float* __restrict__ w, int Cout, const float* __restrict__ bias,
                  int relu, bf16_t* __restrict__ y, int64_t ldy, int64_t begin, int64_t end) {
    extern __shared__ __attribute__((aligned(16))) float wl[];        // [ci][8 * C111_OG]
    constexpr int NO = 8 * C111_OG;
    const int o0 = blockIdx.y * NO, nq = Cin / 8;
    for (int e = threadIdx.x; e < Cin * NO; e += GTB) {
        const int ci = e / NO, co = o0 + (e % NO);
        wl[e] = co < Cout ? w[(int64_t)co * Cin + ci] : 0.f;
    }
    __syncthreads();
    const int64_t i = begin + (int64_t)blockIdx.x * GTB + threadIdx.x;
    if (i >= end) return;
    float acc[NO];
#pragma unroll
    for (int c = 0; c < NO; ++c) acc[c] = 0.f;
    // input groups four at a time: the next four loads are in flight while these are multiplied
    uint4 cur[4], nxt[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) cur[k] = *g8_at(x, ldx, min(k, nq - 1), i);
    for (int q0 = 0; q0 < nq; q0 += 4) {
        if (q0 + 4 < nq) {
#pragma unroll
            for (int k = 0; k < 4; ++k) nxt[k] = *g8_at(x, ldx, min(q0 + 4 + k, nq - 1), i);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (q0 + k >= nq) break;
            float f[8];
            unpack8(cur[k], f);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float* wr = wl + ((q0 + k) * 8 + j) * NO;
#pragma unroll
                for (int c4 = 0; c4 < NO; c4 += 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(wr + c4);
                    acc[c4] += w4.x * f[j]; acc[c4 + 1] += w4.y * f[j]; acc[c4 + 2] += w4.z * f[j]; acc[c4 + 3] += w4.w * f[j];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) cur[k] = nxt[k];
    }
#pragma unroll
    for (int c = 0; c < NO; ++c) {
        const int co = o0 + c;
        if (bias && co < Cout) acc[c] += bias[co];
        if (relu) acc[c] = acc[c] < 0.f ? 0.f : acc[c];
    }
#pragma unroll
    for (int g = 0; g < C111_OG; ++g) {
        if (o0 + 8 * g >= Cout) break;
        if constexpr (OUT_G8) {
            float a8[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) a8[c] = acc[8 * g + c];
            *g8_at(y, ldy, blockIdx.y * C111_OG + g, i) = pack8(a8);
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c)
                if (o0 + 8 * g + c < Cout) y[(int64_t)(o0 + 8 * g + c) * ldy + i] = float_to_bf16(acc[8 * g + c]);
        }
    }
}


// The same operator on the bfloat16 matrix cores, for up to 128 input channels: v_mfma_f32_32x32x16_bf16 contracts
// 16 input channels of 32 particles with 32 outputs, and its B operand -- lane l supplies channels 8 (l / 32) .. + 7
// of particle l % 32 -- IS the 16-byte group of that particle: a lane loads group 2 kb + l / 32 and hands it to the
// instruction untouched.  The fp32 weights are split into a bfloat16 head and a bfloat16 remainder (two instructions
// per 16 channels, the products summed in fp32), so the result keeps the weights to 2^-16.  The vector-ALU kernel above
// needs 2 * Cin * Cout / 64 multiply-add instructions per particle and is bound by them from 32 x 32 on; here the layer
// streams.  A wave takes TILES tiles of 32 particles per round, all their loads in flight before the first product.
typedef __bf16 bf16x8g __attribute__((ext_vector_type(8)));
typedef float floatx16g __attribute__((ext_vector_type(16)));

template <bool OUT_G8, int KB, int MB, int TILES>      // KB blocks of 16 input channels, MB blocks of 32 outputs per workgroup
__global__ void __launch_bounds__(GTB) __attribute__((amdgpu_waves_per_eu(2)))
conv111_g8_mfma_kernel(const bf16_t* __restrict__ x, int64_t ldx, int Cin, const float* __restrict__ w, int Cout,
                       const float* __restrict__ bias, int relu, bf16_t* __restrict__ y, int64_t ldy, int64_t begin, int64_t end) {
    const int lane = threadIdx.x & 63, hi = lane >> 5, col = lane & 31;
    const int o0 = blockIdx.y * 32 * MB, nq = Cin / 8;
    // A operands: lane supplies W[o0 + 32 mb + col][16 kb + 8 hi .. + 7], head and remainder
    bf16x8g ah[MB][KB], al[MB][KB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const int o = o0 + 32 * mb + col, c0 = 16 * kb + 8 * hi;
            float f[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) f[j] = w[(int64_t)min(o, Cout - 1) * Cin + min(c0 + j, Cin - 1)];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float v = (o < Cout && c0 + j < Cin) ? f[j] : 0.f;
                const bf16_t h = float_to_bf16(v);
                const bf16_t l = float_to_bf16(v - bf16_to_float(h));
                ah[mb][kb][j] = __builtin_bit_cast(__bf16, h.bits);
                al[mb][kb][j] = __builtin_bit_cast(__bf16, l.bits);
            }
        }
    // the lane's 16 results of a 32 x 32 block are outputs 8 (r / 4) + 4 hi + r % 4 of particle col
    float bs[MB][16];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int o = o0 + 32 * mb + 8 * (r >> 2) + 4 * hi + (r & 3);
            bs[mb][r] = bias ? bias[min(o, Cout - 1)] : 0.f;
        }
    const int64_t nwave = (int64_t)gridDim.x * (GTB / 64);
    const int64_t wave = (int64_t)blockIdx.x * (GTB / 64) + (threadIdx.x >> 6);
    for (int64_t i0 = begin + wave * (32 * TILES); i0 < end; i0 += nwave * (32 * TILES)) {
        uint4 raw[TILES][KB];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int64_t i = min(i0 + 32 * t + col, end - 1);          // past the end: a particle that exists, never stored
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) raw[t][kb] = *g8_at(x, ldx, min(2 * kb + hi, nq - 1), i);     // (a group past the last: zero weights)
        }
        __builtin_amdgcn_sched_barrier(0);          // all loads in flight before the first matrix instruction
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int64_t i = i0 + 32 * t + col;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                floatx16g acc;
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[r] = bs[mb][r];
#pragma unroll
                for (int kb = 0; kb < KB; ++kb) {
                    const bf16x8g bv = __builtin_bit_cast(bf16x8g, raw[t][kb]);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[mb][kb], bv, acc, 0, 0, 0);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[mb][kb], bv, acc, 0, 0, 0);
                }
                if (i >= end) continue;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int oc = o0 + 32 * mb + 8 * g + 4 * hi;        // the lane's four channels of output group g
                    if (oc >= Cout) continue;
                    float v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) { v[j] = acc[4 * g + j]; if (relu) v[j] = v[j] < 0.f ? 0.f : v[j]; }
                    if constexpr (OUT_G8) {
                        *reinterpret_cast<uint2*>(y + (((int64_t)(oc >> 3) * ldy + i) << 3) + (oc & 4)) =
                            make_uint2((unsigned)float_to_bf16(v[0]).bits | ((unsigned)float_to_bf16(v[1]).bits << 16),
                                       (unsigned)float_to_bf16(v[2]).bits | ((unsigned)float_to_bf16(v[3]).bits << 16));
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (oc + j < Cout) y[(int64_t)(oc + j) * ldy + i] = float_to_bf16(v[j]);
                    }
                }
            }
        }
    }
}

template <bool OUT_G8>
static bool launch_conv111_g8_mfma(const bf16_t* x, int64_t ldx, int Cin, const float* w, int Cout, const float* bias, int relu,
                                   bf16_t* y, int64_t ldy, int64_t b, int64_t e, hipStream_t st) {
    const int kb = (Cin + 15) / 16;
    if (kb > 8) return false;
    const int mb = (Cout > 32 && kb <= 4) ? 2 : 1;
    const int64_t per_block = (int64_t)(GTB / 64) * 32 * (mb == 2 ? 2 : 4);
    dim3 grid((unsigned)std::min<int64_t>((e - b + per_block - 1) / per_block, 256 * 16), (unsigned)((Cout + 32 * mb - 1) / (32 * mb)));
#define APRNET_C111(KB, MB, TILES) hipLaunchKernelGGL((conv111_g8_mfma_kernel<OUT_G8, KB, MB, TILES>), grid, dim3(GTB), 0, st, x, ldx, Cin, w, \
                                                     Cout, bias, relu, y, ldy, b, e)
    if (mb == 2) { if (kb <= 1) APRNET_C111(1, 2, 2); else if (kb <= 2) APRNET_C111(2, 2, 2); else APRNET_C111(4, 2, 2); }
    else if (kb <= 1) APRNET_C111(1, 1, 4);
    else if (kb <= 2) APRNET_C111(2, 1, 4);
    else if (kb <= 4) APRNET_C111(4, 1, 4);
    else APRNET_C111(8, 1, 4);
#undef APRNET_C111
    return true;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {

int aprnet_regroup8_bf16(const uint16_t* x, int64_t ldx, int C, int64_t n, uint16_t* out, int64_t ldo, void* st) {
    if (C <= 0 || n <= 0) return 0;
    if (!x || !out || ldo < n || ldx < n) return fail(APRNET_ERR_INVALID_ARGUMENT, "regroup8: null pointer or row shorter than n");
    dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 1 << 20), (unsigned)((C + 7) / 8));
    hipLaunchKernelGGL(regroup8_kernel, grid, dim3(256), 0, (hipStream_t)st, (const bf16_t*)x, ldx, C, n, (bf16_t*)out, ldo);
    APRNET_LAUNCH_CHECK("regroup8_kernel");
    return 0;
}
int aprnet_ungroup8_bf16(const uint16_t* xg, int64_t ldg, int C, int64_t n, uint16_t* out, int64_t ldo, void* st) {
    if (C <= 0 || n <= 0) return 0;
    if (!xg || !out || ldo < n || ldg < n) return fail(APRNET_ERR_INVALID_ARGUMENT, "ungroup8: null pointer or row shorter than n");
    dim3 grid((unsigned)std::min<int64_t>((n + 255) / 256, 1 << 20), (unsigned)((C + 7) / 8));
    hipLaunchKernelGGL(ungroup8_kernel, grid, dim3(256), 0, (hipStream_t)st, (const bf16_t*)xg, ldg, C, n, (bf16_t*)out, ldo);
    APRNET_LAUNCH_CHECK("ungroup8_kernel");
    return 0;
}
int aprnet_fill_tree_mean_bf16g(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* tree, int64_t ldt, void* st) {
    if (int rc = check_level_delta(p, d, "fill_tree_mean")) return rc;
    if (int rc = check_rows(ldx, p->number_parts(d), "fill_tree_mean (grouped)", "input")) return rc;
    if (int rc = check_rows(ldt, p->tree_parts(d), "fill_tree_mean (grouped)", "tree work space")) return rc;
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    return fill_tree_mean_g8(p, d, (const bf16_t*)x, ldx, C, (bf16_t*)tree, ldt, (hipStream_t)st, nullptr, false);
}
int aprnet_maxpool_fwd_bf16g(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy, void* st) {
    if (int rc = check_level_delta(p, d, "maxpool_forward")) return rc;
    if (C % 8) return fail(APRNET_ERR_INVALID_ARGUMENT, "grouped features hold a multiple of eight channels");
    const int Lc = p->lc(d);
    if (Lc - 1 < p->tree.level_min) return fail(APRNET_ERR_LEVEL_DELTA, "maxpool_forward: nothing left to pool");
    const int64_t n_out = p->number_parts(d + 1), n_copy = p->apr.level_end(Lc - 1);
    if (C <= 0 || n_out <= 0) return 0;
    if (ldy < n_out || ldx < p->number_parts(d)) return fail(APRNET_ERR_INVALID_ARGUMENT, "maxpool_forward: row shorter than the particle count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    hipLaunchKernelGGL(maxpool_g8_kernel, dim3((unsigned)((n_out + GTB - 1) / GTB)), dim3(GTB), 0, (hipStream_t)st,
                       p->d_children, p->n_tree, n_copy, n_out, p->tree.level_begin(Lc - 1), (const bf16_t*)x, ldx, C / 8, (bf16_t*)y, ldy,
                       p->tree_offset(Lc));
    APRNET_LAUNCH_CHECK("maxpool_g8_kernel");
    return 0;
}
int aprnet_upsample_fwd_bf16g(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy, void* st) {
    if (int rc = check_level_delta(p, d, "upsample_const_forward")) return rc;
    if (d <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "UpSampleConst is only implemented for downsampled particles (level_delta > 0)");
    if (C % 8) return fail(APRNET_ERR_INVALID_ARGUMENT, "grouped features hold a multiple of eight channels");
    const int Lc = p->lc(d);
    const int64_t n_in = p->number_parts(d), n_copy = p->apr.level_end(Lc);
    if (C <= 0 || n_in <= 0) return 0;
    if (ldx < n_in || ldy < p->number_parts(d - 1)) return fail(APRNET_ERR_INVALID_ARGUMENT, "upsample_const_forward: row shorter than the particle count");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    const int64_t n_thr = n_copy + 2 * (n_in - n_copy);
    hipLaunchKernelGGL(upsample_g8_kernel, dim3((unsigned)((n_thr + GTB - 1) / GTB)), dim3(GTB), 0, (hipStream_t)st,
                       p->d_children, p->n_tree, n_copy, n_in, p->tree.level_begin(Lc), (const bf16_t*)x, ldx, C / 8, (bf16_t*)y, ldy,
                       p->tree_offset(Lc + 1));
    APRNET_LAUNCH_CHECK("upsample_g8_kernel");
    return 0;
}
int aprnet_conv111_g8_max_cin(void) { return C111_MAX_CIN; }
int aprnet_conv111_fwd_bf16g(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int Cin, const float* w, int S, int Cout,
                             const float* bias, int relu, uint16_t* y, int64_t ldy, int y_grouped, void* st) {
    if (int rc = check_level_delta(p, d, "conv111_forward")) return rc;
    if (Cin <= 0 || Cout <= 0 || S <= 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "conv111_forward: empty channel / stencil count");
    if (Cin % 8 || Cin > C111_MAX_CIN || (y_grouped && Cout % 8))
        return fail(APRNET_ERR_UNSUPPORTED, "conv111_forward (grouped): channel counts must be multiples of eight, at most 256 inputs");
    if (int rc = check_rows(ldx, p->number_parts(d), "conv111_forward (grouped)", "input")) return rc;
    if (int rc = check_rows(ldy, p->number_parts(d), "conv111_forward (grouped)", "output")) return rc;
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    const int Lc = p->lc(d);
    // particles of levels that share a stencil are contiguous: stencil s serves level Lc - s (the downsampled
    // particles sit behind level Lc and take stencil 0 with it), the last stencil every coarser level as well
    for (int s = 0; s < S; ++s) {
        const int l_hi = Lc - s, l_lo = (s == S - 1) ? p->apr.level_min : l_hi;
        if (l_hi < p->apr.level_min) break;
        int64_t b = p->apr.level_begin(std::max(l_lo, p->apr.level_min)), e = p->apr.level_end(l_hi);
        if (s == 0) e = p->number_parts(d);
        if (e <= b) continue;
        dim3 grid((unsigned)((e - b + GTB - 1) / GTB), (unsigned)((Cout + 8 * C111_OG - 1) / (8 * C111_OG)));
        const size_t lds = (size_t)Cin * 8 * C111_OG * sizeof(float);
        const float* ws = w + (int64_t)s * Cout * Cin;
        if (Cin >= 16) {      // also the head of a network (16 -> 3, plane output): it streams its input like the wide layers
            const bool done = y_grouped ? launch_conv111_g8_mfma<true>((const bf16_t*)x, ldx, Cin, ws, Cout, bias, relu, (bf16_t*)y, ldy, b, e, (hipStream_t)st)
                                        : launch_conv111_g8_mfma<false>((const bf16_t*)x, ldx, Cin, ws, Cout, bias, relu, (bf16_t*)y, ldy, b, e, (hipStream_t)st);
            if (done) continue;
        }
        if (y_grouped) hipLaunchKernelGGL(conv111_g8_kernel<true>, grid, dim3(GTB), lds, (hipStream_t)st, (const bf16_t*)x, ldx, Cin, ws, Cout, bias, relu, (bf16_t*)y, ldy, b, e);
        else hipLaunchKernelGGL(conv111_g8_kernel<false>, grid, dim3(GTB), lds, (hipStream_t)st, (const bf16_t*)x, ldx, Cin, ws, Cout, bias, relu, (bf16_t*)y, ldy, b, e);
    }
    APRNET_LAUNCH_CHECK("conv111_g8_kernel");
    return 0;
}

}  // extern "C"
