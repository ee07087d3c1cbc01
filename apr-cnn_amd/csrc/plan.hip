// Plan = device image of one APR: access arrays, child table, convolution tile lists.
// Host side of the C ABI for plan management (include/aprnet_hip.h).
#include "common.hpp"

#include <algorithm>
#include <cstring>
#include <thread>

namespace aprnet {

static thread_local std::string g_last_error;

void set_error(const std::string& msg) { g_last_error = msg; }
int fail(int code, const std::string& msg) { g_last_error = msg; return code; }

template <class F>
static void parallel_for(int n, F f, int serial_below = 64) {
    const int nt = std::max(1u, std::min(16u, std::thread::hardware_concurrency()));
    if (n < serial_below || nt == 1) { for (int i = 0; i < n; ++i) f(i); return; }
    std::vector<std::thread> th;
    for (int t = 0; t < nt; ++t)
        th.emplace_back([=]() { for (int i = t; i < n; i += nt) f(i); });
    for (auto& t : th) t.join();
}

static int copy_access(const aprnet_access_desc* d, HostAccess& h, int lmax_all) {
    if (!d || !d->z_num || !d->x_num || !d->y_num || !d->level_xz_vec || !d->xz_end_vec)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: null access array");
    if (d->level_max + 1 > MAX_LEVELS || d->level_min < 0 || d->level_min > d->level_max)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: level range out of bounds");
    h.level_min = d->level_min; h.level_max = d->level_max; h.n = d->n_particles;
    h.z_num.assign(d->z_num, d->z_num + lmax_all + 1);
    h.x_num.assign(d->x_num, d->x_num + lmax_all + 1);
    h.y_num.assign(d->y_num, d->y_num + lmax_all + 1);
    h.level_xz.assign(d->level_xz_vec, d->level_xz_vec + d->level_max + 2);
    if (h.level_xz[d->level_max + 1] != d->n_rows)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: xz_end_vec length does not match level_xz_vec");
    h.xz_end.assign(d->xz_end_vec, d->xz_end_vec + d->n_rows);
    if (h.xz_end.empty() || h.xz_end[0] != 0 || h.xz_end.back() != d->n_particles)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: xz_end_vec must start at 0 and end at n_particles");
    // the convolution kernels address a channel plane with 32-bit byte offsets: 2^30 elements of 4 bytes
    // (conv entry points check the element size of the call, check_plane_size)
    if (d->n_particles >= (1ull << 30))
        return fail(APRNET_ERR_UNSUPPORTED, "plan_create: 2^30 or more particles per access");
    if (d->n_particles && !d->y_vec) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: null y_vec with particles present");
    // The arrays may come from a file: everything the kernels index with is checked here once, so that a damaged
    // state is an error code and not an out-of-range access on the GPU.
    for (int l = 0; l <= lmax_all; ++l)
        if (h.z_num[l] < 1 || h.x_num[l] < 1 || h.y_num[l] < 1 || h.y_num[l] > 65536)
            return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: level dimensions must lie in 1..65536 (y) and be positive");
    if (h.level_xz[d->level_min] < 1) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: level_xz_vec must leave the leading sentinel row");
    for (int l = d->level_min; l <= d->level_max; ++l)
        if (h.level_xz[l + 1] < h.level_xz[l] || h.level_xz[l + 1] - h.level_xz[l] != (uint64_t)h.z_num[l] * (uint64_t)h.x_num[l])
            return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: level_xz_vec does not match z_num * x_num of level " + std::to_string(l));
    std::vector<int> bad_level(d->level_max + 1, 0);
    for (int l = d->level_min; l <= d->level_max; ++l) {
        const uint64_t r0 = h.level_xz[l], r1 = h.level_xz[l + 1];
        const int yn = h.y_num[l];
        const uint64_t* xz = h.xz_end.data();
        const uint16_t* yv = d->y_vec;
        const uint64_t n = d->n_particles;
        std::vector<int> bad(16, 0);
        parallel_for(16, [&](int t) {
            for (uint64_t r = r0 + (uint64_t)t; r < r1; r += 16) {
                const uint64_t b = xz[r - 1], e = xz[r];
                if (e < b || e > n) { bad[t] = 1; return; }
                for (uint64_t i = b; i < e; ++i)
                    if ((int)yv[i] >= yn || (i > b && yv[i] <= yv[i - 1])) { bad[t] = 2; return; }
            }
        }, 1);
        for (int t = 0; t < 16; ++t) bad_level[l] = std::max(bad_level[l], bad[t]);
        if (bad_level[l] == 1)
            return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: xz_end_vec must be non-decreasing and end within n_particles (level " + std::to_string(l) + ")");
        if (bad_level[l] == 2)
            return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: y_vec must ascend strictly within a row and stay below y_num (level " + std::to_string(l) + ")");
    }
    // rows below level_min (none by construction of level_xz_vec) and the sentinel hold no particles
    if (h.xz_end[h.level_xz[d->level_min] - 1] != 0)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: rows before level_min must be empty");
    if (d->n_particles) h.y.assign(d->y_vec, d->y_vec + d->n_particles);
    return 0;
}

static void fill_dev(const HostAccess& h, AccessDev& d, const void* xz, const void* y, int lmax_all) {
    std::memset(&d, 0, sizeof(d));
    d.xz_end = (const uint64_t*)xz; d.y = (const uint16_t*)y;
    d.level_min = h.level_min; d.level_max = h.level_max;
    for (int l = 0; l <= lmax_all; ++l) { d.z_num[l] = h.z_num[l]; d.x_num[l] = h.x_num[l]; d.y_num[l] = h.y_num[l]; }
    for (int l = 0; l <= h.level_max + 1; ++l) d.level_xz[l] = h.level_xz[l];
    for (int l = h.level_max + 2; l <= MAX_LEVELS; ++l) d.level_xz[l] = h.level_xz[h.level_max + 1];
}


// children[s][t], s = 4*dz + 2*dx + dy: the merge walk of helpers.hpp:185-194 done once, from the
// parents' side, for particles and for tree nodes.
static void build_children(const HostAccess& apr, const HostAccess& tree, std::vector<int32_t>& ch) {
    const int64_t T = (int64_t)tree.n;
    ch.assign((size_t)8 * T, NO_CHILD);
    for (int l = tree.level_min; l <= tree.level_max; ++l) {
        const int cl = l + 1;
        const int zn = tree.z_num[l], xn = tree.x_num[l];
        const int czn = tree.z_num[cl], cxn = tree.x_num[cl];
        const bool apr_has = cl >= apr.level_min && cl <= apr.level_max;
        const bool tree_has = cl <= tree.level_max;
        parallel_for(zn, [&](int z) {
            for (int x = 0; x < xn; ++x) {
                const uint64_t prow = tree.row(l, z, x);
                const int64_t pb = (int64_t)tree.xz_end[prow - 1], pe = (int64_t)tree.xz_end[prow];
                if (pb == pe) continue;
                for (int dz = 0; dz < 2; ++dz) {
                    const int cz = 2 * z + dz; if (cz >= czn) continue;
                    for (int dx = 0; dx < 2; ++dx) {
                        const int cx = 2 * x + dx; if (cx >= cxn) continue;
                        const int s0 = 4 * dz + 2 * dx;
                        if (apr_has) {
                            const uint64_t r = apr.row(cl, cz, cx);
                            int64_t p = pb;
                            for (int64_t c = (int64_t)apr.xz_end[r - 1]; c < (int64_t)apr.xz_end[r]; ++c) {
                                const int yp = apr.y[c] >> 1;
                                while (p < pe && tree.y[p] < yp) ++p;
                                if (p < pe && tree.y[p] == yp) ch[(size_t)(s0 + (apr.y[c] & 1)) * T + p] = (int32_t)c;
                            }
                        }
                        if (tree_has) {
                            const uint64_t r = tree.row(cl, cz, cx);
                            int64_t p = pb;
                            for (int64_t c = (int64_t)tree.xz_end[r - 1]; c < (int64_t)tree.xz_end[r]; ++c) {
                                const int yp = tree.y[c] >> 1;
                                while (p < pe && tree.y[p] < yp) ++p;
                                if (p < pe && tree.y[p] == yp) ch[(size_t)(s0 + (tree.y[c] & 1)) * T + p] = ~(int32_t)c;
                            }
                        }
                    }
                }
            }
        });
    }
}

bool stream_is_capturing(hipStream_t st) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) { (void)hipGetLastError(); return false; }
    return cs != hipStreamCaptureStatusNone;
}

void plan_scratch_done(aprnet_plan* p, hipStream_t st) {
    if (stream_is_capturing(st)) { p->scratch_event_recorded = false; return; }   // inside a graph the caller orders its streams
    if (!p->ev_scratch && hipEventCreateWithFlags(&p->ev_scratch, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError(); p->ev_scratch = nullptr; p->scratch_event_recorded = false;
        (void)hipStreamSynchronize(st);          // no event to hand over with: finish the work instead
        return;
    }
    p->scratch_event_recorded = hipEventRecord(p->ev_scratch, st) == hipSuccess;
    if (!p->scratch_event_recorded) { (void)hipGetLastError(); (void)hipStreamSynchronize(st); }
}

int plan_scratch(aprnet_plan* p, size_t bytes, hipStream_t st) {
    const bool capturing = stream_is_capturing(st);
    // a second stream takes the buffer over only after the first is done with it: a device-side wait for the event
    // that the previous call recorded behind its kernels
    if (p->scratch_stream_valid && p->scratch_stream != st && p->scratch_event_recorded && !capturing)
        APRNET_HIP_CHECK(hipStreamWaitEvent(st, p->ev_scratch, 0));
    p->scratch_stream = st; p->scratch_stream_valid = true;
    if (bytes > p->scratch_bytes) {
        if (capturing)
            return fail(APRNET_ERR_UNSUPPORTED, "the plan's scratch buffer would have to grow while the stream is capturing: call "
                                                "aprnet_plan_reserve, or run this call once, before the capture");
        if (p->d_scratch) {
            if (p->scratch_in_graph) p->retired.push_back(p->d_scratch);     // a graph may replay into it: keep it until destroy
            else {
                // nothing may still read the old buffer: this stream's work, and the last user's (another stream's)
                APRNET_HIP_CHECK(hipStreamSynchronize(st));
                if (p->scratch_event_recorded) APRNET_HIP_CHECK(hipEventSynchronize(p->ev_scratch));
                APRNET_HIP_CHECK(hipFree(p->d_scratch));
            }
        }
        p->d_scratch = nullptr; p->scratch_bytes = 0; p->scratch_in_graph = false;
        APRNET_HIP_CHECK(hipMalloc(&p->d_scratch, bytes));
        p->scratch_bytes = bytes;
    }
    if (capturing) p->scratch_in_graph = true;
    return 0;
}

int get_tiles(aprnet_plan* plan, int level_delta, int TZ, int TX, TileList* out, hipStream_t st, int halo) {
    auto key = std::make_tuple(level_delta, TZ, TX, halo);
    auto it = plan->tiles.find(key);
    if (it != plan->tiles.end()) { *out = it->second; return 0; }
    if (stream_is_capturing(st))
        return fail(APRNET_ERR_UNSUPPORTED, "the first convolution at a level delta builds the plan's tile lists (allocates and "
                                            "copies): run it once before capturing the stream");
    const HostAccess& apr = plan->apr; const HostAccess& tree = plan->tree;
    const int Lc = plan->lc(level_delta);
    std::vector<ConvTile> tiles;
    TileList tl;
    // finest level first: it holds most of the work, the coarse levels fill the tail of the launch
    for (int l = Lc; l >= apr.level_min; --l) {
        tl.level_begin[l] = (int)tiles.size();
        const bool with_tree = (l == Lc && l < apr.level_max);
        const int zn = apr.z_num[l], xn = apr.x_num[l];
        for (int z0 = 0; z0 < zn; z0 += TZ)
            for (int x0 = 0; x0 < xn; x0 += TX) {
                bool any = false;
                for (int z = std::max(z0 - halo, 0); z < std::min(z0 + TZ + halo, zn) && !any; ++z) {
                    const int xa = std::max(x0 - halo, 0), x1 = std::min(x0 + TX + halo, xn) - 1;
                    // rows xa..x1 of one z are adjacent in the row table: one range test
                    const uint64_t ra = apr.row(l, z, xa), rb = apr.row(l, z, x1);
                    any = apr.xz_end[rb] > apr.xz_end[ra - 1];
                    if (!any && with_tree) {
                        const uint64_t ta = tree.row(l, z, xa), tb = tree.row(l, z, x1);
                        any = tree.xz_end[tb] > tree.xz_end[ta - 1];
                    }
                }
                if (any) tiles.push_back(ConvTile{l, z0, x0, 0});
            }
        tl.level_count[l] = (int)tiles.size() - tl.level_begin[l];
    }
    tl.n = (int)tiles.size();
    if (tl.n) {
        APRNET_HIP_CHECK(hipMalloc((void**)&tl.d_tiles, tiles.size() * sizeof(ConvTile)));
        APRNET_HIP_CHECK(hipMemcpy(tl.d_tiles, tiles.data(), tiles.size() * sizeof(ConvTile), hipMemcpyHostToDevice));
    }
    plan->tiles[key] = tl;
    *out = tl;
    return 0;
}

}  // namespace aprnet

using namespace aprnet;

extern "C" {

const char* aprnet_last_error(void) { return g_last_error.c_str(); }

int aprnet_plan_create(const aprnet_access_desc* apr, const aprnet_access_desc* tree, int device, aprnet_plan** out) {
    if (!out) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: null output");
    *out = nullptr;
    if (!apr || !tree) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: null access descriptor");
    if (tree->level_max != apr->level_max - 1 || tree->level_min > apr->level_min - 1)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_create: the tree must span levels <= level_min-1 .. level_max-1");
    aprnet_plan* p = new aprnet_plan();
    p->device = device;
    const int lmax_all = apr->level_max;
    int rc = copy_access(apr, p->apr, lmax_all);
    if (!rc) rc = copy_access(tree, p->tree, lmax_all);
    if (rc) { delete p; return rc; }
    p->n_apr = (int64_t)p->apr.n; p->n_tree = (int64_t)p->tree.n;
    // copy_access has checked that y ascends strictly per row: build_children and the staging code rely on it
    std::vector<int32_t> children;
    build_children(p->apr, p->tree, children);

    if (hipError_t e = hipSetDevice(device); e != hipSuccess) {
        delete p;
        return fail(APRNET_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
    }
    auto upload = [&](void** dst, const void* src, size_t bytes) -> int {
        APRNET_HIP_CHECK(hipMalloc(dst, std::max<size_t>(bytes, 16)));
        if (bytes) APRNET_HIP_CHECK(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return 0;
    };
    rc = upload(&p->d_apr_xz, p->apr.xz_end.data(), p->apr.xz_end.size() * 8);
    if (!rc) rc = upload(&p->d_apr_y, p->apr.y.data(), p->apr.y.size() * 2);
    if (!rc) rc = upload(&p->d_tree_xz, p->tree.xz_end.data(), p->tree.xz_end.size() * 8);
    if (!rc) rc = upload(&p->d_tree_y, p->tree.y.data(), p->tree.y.size() * 2);
    if (!rc) rc = upload((void**)&p->d_children, children.data(), children.size() * 4);
    if (rc) { aprnet_plan_destroy(p); return rc; }
    fill_dev(p->apr, p->dapr, p->d_apr_xz, p->d_apr_y, lmax_all);
    fill_dev(p->tree, p->dtree, p->d_tree_xz, p->d_tree_y, lmax_all);
    // the host keeps only the row tables (for level ranges and tile lists), not y
    *out = p;
    return 0;
}

void aprnet_plan_destroy(aprnet_plan* p) {
    if (!p) return;
    (void)hipSetDevice(p->device);
    for (void* q : {p->d_apr_xz, p->d_apr_y, p->d_tree_xz, p->d_tree_y, (void*)p->d_children})
        if (q) (void)hipFree(q);
    for (auto& kv : p->tiles) if (kv.second.d_tiles) (void)hipFree(kv.second.d_tiles);
    if (p->d_scratch) (void)hipFree(p->d_scratch);
    for (void* q : p->retired) (void)hipFree(q);
    for (auto& kv : p->lists) free_lists(kv.second);
    for (auto& kv : p->faces) free_face_lists(kv.second);
    for (auto& kv : p->need) free_need_lists(kv.second);
    if (p->side) { (void)hipStreamSynchronize(p->side); (void)hipStreamDestroy(p->side); }
    if (p->ev_fork) (void)hipEventDestroy(p->ev_fork);
    if (p->ev_join) (void)hipEventDestroy(p->ev_join);
    if (p->ev_scratch) (void)hipEventDestroy(p->ev_scratch);
    delete p;
}

int64_t aprnet_number_parts(const aprnet_plan* p, int level_delta) { return p ? p->number_parts(level_delta) : -1; }
int64_t aprnet_tree_offset(const aprnet_plan* p, int level) { return p ? p->tree_offset(level) : 0; }
int64_t aprnet_tree_parts(const aprnet_plan* p, int level_delta) { return p ? p->tree_parts(level_delta) : -1; }

int aprnet_plan_reserve(aprnet_plan* p, int64_t bytes, void* stream) {
    if (!p || bytes < 0) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_reserve: null plan or negative size");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    return plan_scratch(p, (size_t)bytes, (hipStream_t)stream);
}

int aprnet_plan_children(const aprnet_plan* p, int32_t* out_host) {
    if (!p || !out_host) return fail(APRNET_ERR_INVALID_ARGUMENT, "plan_children: null argument");
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    if (p->n_tree) APRNET_HIP_CHECK(hipMemcpy(out_host, p->d_children, (size_t)8 * p->n_tree * 4, hipMemcpyDeviceToHost));
    return 0;
}

}  // extern "C"
