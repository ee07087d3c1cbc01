// Which tree nodes a convolution reads.
//
// A stencil convolution at a level delta reads the mean-filled tree only where a staged row of a tile below the
// current maximum level crosses a region that is resolved more finely: the items of the plan's window lists that carry
// ITEM_TREE.  On a typical APR most particles sit on the finest level and those regions' interiors are never read, so
// filling the whole tree per convolution (the reference does it per input channel, conv.hpp:109-110) is mostly wasted
// traffic: the full-resolution layers of a network re-read their whole input for it.  This file derives, once per plan,
// level delta and stencil, the set of tree nodes that must hold a mean: the nodes the lists name plus all their
// descendants inside the tree work space (a node's mean needs its children's), as one ascending index list per level.
#include "conv_common.hpp"

#include <algorithm>

namespace aprnet {

__global__ void need_zero_kernel(unsigned char* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

__global__ void need_mark_items_kernel(const int* __restrict__ item_idx, const unsigned short* __restrict__ item_pos, int64_t n_items,
                                       int64_t n_mark, unsigned char* __restrict__ mark) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_items; i += (int64_t)gridDim.x * blockDim.x) {
        const unsigned pos = item_pos[i];
        if (pos == 0xffffu || !(pos & ITEM_TREE)) continue;
        const int64_t t = item_idx[i];
        if (t >= 0 && t < n_mark) mark[t] = 1;
    }
}

// marked nodes of [t_begin, t_end) mark their tree children (all one level finer), when those lie below n_mark
__global__ void need_close_level_kernel(const int32_t* __restrict__ children, int64_t n_tree, int64_t t_begin, int64_t t_end,
                                        int64_t n_mark, unsigned char* __restrict__ mark) {
    const int64_t t = t_begin + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= t_end || !mark[t]) return;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int32_t v = children[(int64_t)s * n_tree + t];
        if (v < 0 && v != NO_CHILD && (int64_t)~v < n_mark) mark[~v] = 1;
    }
}

void free_need_lists(NeedLists& nl) {
    if (nl.d_nodes) (void)hipFree(nl.d_nodes);
    nl = NeedLists{};
}

// Needed tree nodes of the forward convolution at `level_delta` with stencil `code`, from its window lists `wl`.
// Built on first use (synchronises the stream, allocates, copies the marks to the host once), then served from the plan.
int get_need_lists(aprnet_plan* p, int level_delta, int code, const WinLists& wl, NeedLists* out, hipStream_t st) {
    auto key = std::make_pair(level_delta, code);
    auto it = p->need.find(key);
    if (it != p->need.end()) {
        *out = it->second;
        return it->second.unavailable ? fail(APRNET_ERR_UNSUPPORTED, "needed-node lists are not available for this plan") : 0;
    }
    if (stream_is_capturing(st))
        return fail(APRNET_ERR_UNSUPPORTED, "needed-node lists are built on the first call at a level delta: run it once before capturing");
    NeedLists nl{};
    NeedLists none{}; none.unavailable = true;
    p->need[key] = none;                 // replaced below when the build succeeds
    const int Lc = p->lc(level_delta);
    const int64_t n_mark = p->tree_parts(level_delta);           // nodes of levels < Lc: the tree work space
    const int l_top = std::min(Lc - 1, p->tree.level_max);
    if (n_mark > 0 && n_mark < ((int64_t)1 << 31) && wl.n_items > 0) {
        unsigned char* d_mark = nullptr;
        APRNET_HIP_CHECK(hipMalloc((void**)&d_mark, (size_t)n_mark));
        hipLaunchKernelGGL(need_zero_kernel, dim3((unsigned)std::min<int64_t>((n_mark + 255) / 256, 65535)), dim3(256), 0, st, d_mark, n_mark);
        hipLaunchKernelGGL(need_mark_items_kernel, dim3((unsigned)std::min<int64_t>((wl.n_items + 255) / 256, 65535)), dim3(256), 0, st,
                           wl.d_item_idx, wl.d_item_pos, wl.n_items, n_mark, d_mark);
        for (int l = p->tree.level_min; l < l_top; ++l) {        // coarse to fine: a level's marks are final when it is visited
            const int64_t b = p->tree.level_begin(l), e = p->tree.level_end(l);
            if (e <= b) continue;
            hipLaunchKernelGGL(need_close_level_kernel, dim3((unsigned)((e - b + 255) / 256)), dim3(256), 0, st, p->d_children, p->n_tree,
                               b, e, n_mark, d_mark);
        }
        hipError_t e1 = hipGetLastError();
        if (e1 != hipSuccess) { (void)hipFree(d_mark); return fail(APRNET_ERR_HIP, std::string("need lists: ") + hipGetErrorString(e1)); }
        std::vector<unsigned char> mark((size_t)n_mark);
        hipError_t e2 = hipStreamSynchronize(st);
        if (e2 == hipSuccess) e2 = hipMemcpy(mark.data(), d_mark, (size_t)n_mark, hipMemcpyDeviceToHost);
        (void)hipFree(d_mark);
        if (e2 != hipSuccess) return fail(APRNET_ERR_HIP, std::string("need lists: ") + hipGetErrorString(e2));
        std::vector<int32_t> nodes;
        for (int l = l_top; l >= p->tree.level_min; --l) {
            const int64_t b = p->tree.level_begin(l), e = std::min<int64_t>(p->tree.level_end(l), n_mark);
            nl.off[l] = (int64_t)nodes.size();
            for (int64_t t = b; t < e; ++t) if (mark[(size_t)t]) nodes.push_back((int32_t)t);
            nl.cnt[l] = (int64_t)nodes.size() - nl.off[l];
            // a level that is needed almost entirely is cheaper to fill whole (coalesced, no index list)
            nl.whole[l] = e > b && nl.cnt[l] * 10 >= (e - b) * 6;
        }
        nl.n_nodes = (int64_t)nodes.size();
        if (!nodes.empty()) {
            APRNET_HIP_CHECK(hipMalloc((void**)&nl.d_nodes, nodes.size() * sizeof(int32_t)));
            hipError_t e3 = hipMemcpy(nl.d_nodes, nodes.data(), nodes.size() * sizeof(int32_t), hipMemcpyHostToDevice);
            if (e3 != hipSuccess) { free_need_lists(nl); return fail(APRNET_ERR_HIP, std::string("need lists: ") + hipGetErrorString(e3)); }
        }
    } else if (n_mark >= ((int64_t)1 << 31)) {
        return fail(APRNET_ERR_UNSUPPORTED, "needed-node lists: more than 2^31 tree nodes");
    }
    p->need[key] = nl;
    *out = nl;
    return 0;
}

}  // namespace aprnet
