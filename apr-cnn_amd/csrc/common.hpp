// Shared declarations of the HIP operator library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <climits>
#include <map>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/aprnet_hip.h"

namespace aprnet {

constexpr int MAX_LEVELS = 18;          // levels 0..17 (y_vec is uint16 -> dims <= 65536 -> level_max <= 16)
constexpr int32_t NO_CHILD = INT32_MIN; // child-table sentinel: cell outside the image

// Device view of one linear access structure; passed to kernels by value.
struct AccessDev {
    const uint64_t* xz_end;             // device, row table with leading 0
    const uint16_t* y;                  // device
    uint64_t level_xz[MAX_LEVELS + 1];
    int32_t z_num[MAX_LEVELS], x_num[MAX_LEVELS], y_num[MAX_LEVELS];
    int32_t level_min, level_max;

    __device__ __forceinline__ uint64_t row(int l, int z, int x) const { return level_xz[l] + (uint64_t)z * x_num[l] + x; }
};

struct HostAccess {
    int level_min = 0, level_max = 0;
    std::vector<int32_t> z_num, x_num, y_num;
    std::vector<uint64_t> level_xz, xz_end;
    std::vector<uint16_t> y;
    uint64_t n = 0;
    uint64_t row(int l, int z, int x) const { return level_xz[l] + (uint64_t)z * x_num[l] + x; }
    // first index of level l / one past the last index of level l (levels outside the range are empty)
    int64_t level_begin(int l) const {
        if (l < level_min) return 0;
        if (l > level_max) return (int64_t)n;
        return (int64_t)xz_end[level_xz[l] - 1];
    }
    int64_t level_end(int l) const {
        if (l < level_min) return 0;
        if (l > level_max) return (int64_t)n;
        return (int64_t)xz_end[level_xz[l + 1] - 1];
    }
};

// bfloat16 as a storage type: kernels load it into fp32, compute in fp32 and round to nearest even on store.
struct bf16_t { uint16_t bits; };
__host__ __device__ inline float bf16_to_float(bf16_t v) { return __builtin_bit_cast(float, (uint32_t)v.bits << 16); }
__host__ __device__ inline bf16_t float_to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return bf16_t{__builtin_bit_cast(uint16_t, (__bf16)f)};      // v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN
#endif
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t{(uint16_t)((u >> 16) | 0x40u)};      // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return bf16_t{(uint16_t)(u >> 16)};
}
// element type -> the type it is computed in, with the conversions of a load and a store
template <typename T> struct Num {
    typedef T acc;
    static __host__ __device__ __forceinline__ acc ld(T v) { return v; }
    static __host__ __device__ __forceinline__ T st(acc v) { return v; }
};
template <> struct Num<bf16_t> {
    typedef float acc;
    static __host__ __device__ __forceinline__ float ld(bf16_t v) { return bf16_to_float(v); }
    static __host__ __device__ __forceinline__ bf16_t st(float v) { return float_to_bf16(v); }
};

struct ConvTile { int32_t level, z0, x0, pad; };

struct TileList {
    ConvTile* d_tiles = nullptr; int n = 0;
    int level_begin[MAX_LEVELS + 1] = {};   // tiles are sorted finest level first: level l owns
    int level_count[MAX_LEVELS + 1] = {};   // [level_begin[l], level_begin[l] + level_count[l])
};

// Precomputed window lists of the forward convolution (lists.hip), device arrays owned by the plan.
struct WinLists {
    int* d_tile_win = nullptr;                  // [n_tiles + 1]
    int4* d_win = nullptr;                      // [n_win] {first item, items, first column, columns}
    int* d_item_idx = nullptr; unsigned short* d_item_pos = nullptr;
    int* d_col_idx = nullptr; unsigned short* d_col_pos = nullptr;
    int n_win = 0; int64_t n_items = 0, n_cols = 0;
    bool unavailable = false;                   // building them failed once (no memory, too many entries): do not retry
    // the levels that have windows, in window order (finest first): first window and level of each
    int n_lv = 0; int lv_first[MAX_LEVELS] = {}; int lv_level[MAX_LEVELS] = {};
};

// Tree nodes whose mean a convolution reads (need.hip): per tree level an ascending list of node indices in `d_nodes`.
struct NeedLists {
    int32_t* d_nodes = nullptr;
    int64_t n_nodes = 0;
    int64_t off[MAX_LEVELS + 1] = {}, cnt[MAX_LEVELS + 1] = {};   // first entry and count of a level's list
    bool whole[MAX_LEVELS + 1] = {};                               // the level is needed (almost) entirely: fill it whole
    bool unavailable = false;                                      // building them failed once: do not retry
};

// Particles that stick out of a far face of the next finer level, with the (output, tap) pairs that read them
// (faces.hip); device arrays owned by the plan.
struct FaceLists {
    int n_part = 0;
    int* d_part_idx = nullptr;                  // [n_part] index of the particle in the input gradient
    int* d_part_level = nullptr;                // [n_part] level of the outputs that read it (its own level + 1)
    int* d_pair_begin = nullptr;                // [n_part + 1]
    int* d_pair_out = nullptr;                  // [pairs] index into the output gradient
    unsigned char* d_pair_tap = nullptr;        // [pairs]
};

}  // namespace aprnet

struct aprnet_plan {
    int device = 0;
    aprnet::HostAccess apr, tree;
    aprnet::AccessDev dapr{}, dtree{};
    void* d_apr_xz = nullptr; void* d_apr_y = nullptr; void* d_tree_xz = nullptr; void* d_tree_y = nullptr;
    int32_t* d_children = nullptr;      // [8][n_tree], slot-major
    int64_t n_tree = 0, n_apr = 0;
    std::map<std::tuple<int, int, int, int>, aprnet::TileList> tiles;   // (level_delta, TZ, TX, halo) -> row groups
    void* d_scratch = nullptr; size_t scratch_bytes = 0;          // re-laid-out weights of the call in flight
    bool scratch_in_graph = false;                                // the buffer was handed out while its stream was capturing
    std::vector<void*> retired;                                   // outgrown buffers that a captured graph may address: freed at destroy
    // Hand-over of the buffer between streams: the last call that used it recorded ev_scratch behind its kernels, and a
    // call on another stream waits for that event on the device (no host synchronisation).  scratch_stream is kept for
    // comparison only; it is never passed to a HIP call, so the stream it named may have been destroyed since.
    hipStream_t scratch_stream = nullptr;
    hipEvent_t ev_scratch = nullptr;
    bool scratch_stream_valid = false, scratch_event_recorded = false;
    std::map<std::pair<int, int>, aprnet::WinLists> lists;        // (level_delta, stencil code) -> window lists
    std::map<std::pair<int, int>, aprnet::FaceLists> faces;       // (level_delta, stencil code) -> far-face particles
    std::map<std::pair<int, int>, aprnet::NeedLists> need;        // (level_delta, stencil code) -> tree nodes the convolution reads
    // second stream of the convolution backward (weight gradient next to input gradient), with its fork / join events
    hipStream_t side = nullptr; hipEvent_t ev_fork = nullptr, ev_join = nullptr;

    int lc(int level_delta) const { return apr.level_max - level_delta; }
    int64_t number_parts(int level_delta) const {
        const int L = lc(level_delta);
        int64_t n = apr.level_end(L);
        if (L <= tree.level_max && L >= tree.level_min) n += tree.level_end(L) - tree.level_begin(L);
        return n;
    }
    int64_t tree_offset(int level) const { return apr.level_end(level) - tree.level_begin(level); }
    int64_t tree_parts(int level_delta) const { const int L = lc(level_delta); return L >= 1 ? tree.level_end(L - 1) : 0; }
};

namespace aprnet {

void set_error(const std::string& msg);
int fail(int code, const std::string& msg);
// non-empty row groups for the convolution at `level_delta` (built on first use, cached in the plan)
// `halo` > 0 also lists the row groups that lie within that many rows of a non-empty one
// (allocates and copies on first use: refused with APRNET_ERR_UNSUPPORTED while `st` is capturing)
int get_tiles(aprnet_plan* plan, int level_delta, int TZ, int TX, TileList* out, hipStream_t st, int halo = 0);
// true while `st` records into a graph (allocation, synchronous copies and stream synchronisation are not allowed then)
bool stream_is_capturing(hipStream_t st);
int get_lists(aprnet_plan* plan, int level_delta, int code, const TileList& tl, WinLists* out, hipStream_t st, bool dx = false);
void free_lists(WinLists& wl);
int get_face_lists(aprnet_plan* plan, int level_delta, int code, FaceLists* out, hipStream_t st);
void free_face_lists(FaceLists& fl);
int get_need_lists(aprnet_plan* plan, int level_delta, int code, const WinLists& wl, NeedLists* out, hipStream_t st);
void free_need_lists(NeedLists& nl);
// Makes plan->d_scratch at least `bytes` large for a call on `st` (contents are lost when it grows).  A buffer that a
// captured graph may address is never freed before the plan is destroyed; growth while `st` is capturing is refused
// with APRNET_ERR_UNSUPPORTED (reserve first: aprnet_plan_reserve, or run the call once outside the capture).  A call on
// another stream than the previous one first waits for that stream, so that two streams cannot overwrite each other's
// packed weights (under capture the caller must have ordered the streams, as for any input of the graph).
int plan_scratch(aprnet_plan* plan, size_t bytes, hipStream_t st);
// Records "this call is done with the scratch buffer" on `st` (after the last kernel that reads it was launched).
void plan_scratch_done(aprnet_plan* plan, hipStream_t st);
// A call's hold on the scratch buffer: acquire() is plan_scratch(); the destructor records the hand-over event, on every
// way out of the call.  Declare it before anything that enqueues work at scope exit (the side-stream join), so that
// its destructor runs last.
struct ScratchLease {
    aprnet_plan* plan = nullptr; hipStream_t st = nullptr;
    int acquire(aprnet_plan* p, size_t bytes, hipStream_t s) {
        const int rc = plan_scratch(p, bytes, s);
        if (!rc) { plan = p; st = s; }
        return rc;
    }
    ~ScratchLease() { if (plan) plan_scratch_done(plan, st); }
    ScratchLease() = default;
    ScratchLease(const ScratchLease&) = delete;
    ScratchLease& operator=(const ScratchLease&) = delete;
};

#define APRNET_HIP_CHECK(expr)                                                                                  \
    do {                                                                                                        \
        hipError_t e_ = (expr);                                                                                 \
        if (e_ != hipSuccess)                                                                                   \
            return aprnet::fail(APRNET_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));             \
    } while (0)

#define APRNET_LAUNCH_CHECK(name)                                                                               \
    do {                                                                                                        \
        hipError_t e_ = hipGetLastError();                                                                      \
        if (e_ != hipSuccess)                                                                                   \
            return aprnet::fail(APRNET_ERR_HIP, std::string("launch of ") + name + ": " + hipGetErrorString(e_)); \
    } while (0)

// buffer loads of the convolution kernels use 32-bit byte offsets inside a channel plane
inline int check_plane_size(const aprnet_plan* p, int d, size_t elem, const char* who) {
    if ((uint64_t)p->number_parts(d) * elem >= (1ull << 32) || (uint64_t)p->tree_parts(d) * elem >= (1ull << 32))
        return fail(APRNET_ERR_UNSUPPORTED, std::string(who) + ": a channel plane of this element size exceeds 4 GiB");
    return 0;
}

// a channel plane (or group) must hold at least the `need` elements the kernels address: a shorter row would turn into
// an out-of-range device access instead of an error code
inline int check_rows(int64_t ld, int64_t need, const char* who, const char* what) {
    if (ld < need)
        return fail(APRNET_ERR_INVALID_ARGUMENT, std::string(who) + ": " + what + " holds " + std::to_string(ld) +
                    " elements per channel, the APR has " + std::to_string(need) + " at this level delta");
    return 0;
}

inline int check_level_delta(const aprnet_plan* p, int d, const char* who) {
    if (!p) return fail(APRNET_ERR_INVALID_ARGUMENT, std::string(who) + ": null plan");
    // CHECK_LEVEL_DELTA(dlvl, tree.level_max()+1): cuda/src/common.hpp:17, wrap_conv_gpu.hpp:46
    if (d < 0 || d >= p->tree.level_max + 1)
        return fail(APRNET_ERR_LEVEL_DELTA, std::string(who) + ": level delta " + std::to_string(d) +
                    " is too large for APR with maximum level " + std::to_string(p->apr.level_max));
    return 0;
}

}  // namespace aprnet
