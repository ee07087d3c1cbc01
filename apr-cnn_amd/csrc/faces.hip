// Input gradient of the particles that stick out of the far faces of a level.
//
// A particle one level coarser than a tile fills the 2 x 2 x 2 cells it covers (helpers.hpp:381-399).  The input
// gradient kernel gives such a particle ONE column that reads the box-summed output gradient (conv_mfma.hip), which
// needs all eight cells to exist.  Where a level has an odd size, the particles on its far faces cover cells outside
// the image; the forward pass never read those cells (zero_boundary, helpers.hpp:481-502), so only the existing
// cells count.  There are few such particles (a 2-D set), and they are handled here, away from the main kernel,
// so that every element of the input gradient receives at most two atomic contributions there (same-level term and
// box term: the sum of two values onto zero does not depend on their order) and the gradient repeats bit for bit.
//
// Built once per plan, level delta and stencil on the host: for each such particle the list of (output position,
// tap) pairs through which the forward pass read it.  The kernel sums
//     gx[ci][p] += sum_pairs sum_co w[s][co][ci][tap] * gy[co][out]
// one workgroup per particle, one thread per input channel, pairs and output channels in list order.
#include "common.hpp"

#include <algorithm>

namespace aprnet {

// index of the particle at (row, y) of an access, or -1
static int64_t find_in_row(const HostAccess& h, int l, int z, int x, int y) {
    const uint64_t row = h.row(l, z, x);
    const uint16_t* b = h.y.data() + h.xz_end[row - 1];
    const uint16_t* e = h.y.data() + h.xz_end[row];
    const uint16_t* it = std::lower_bound(b, e, (uint16_t)y);
    return (it != e && *it == (uint16_t)y) ? (int64_t)(it - h.y.data()) : -1;
}

int get_face_lists(aprnet_plan* p, int d, int code, FaceLists* out, hipStream_t st) {
    auto key = std::make_pair(d, code);
    auto it = p->faces.find(key);
    if (it != p->faces.end()) { *out = it->second; return 0; }
    if (stream_is_capturing(st))
        return fail(APRNET_ERR_UNSUPPORTED, "the first convolution backward at a level delta builds the plan's face lists "
                                            "(allocates and copies): run it once before capturing the stream");
    const HostAccess& apr = p->apr; const HostAccess& tree = p->tree;
    const int kz = code / 100, kx = (code / 10) % 10, ky = code % 10;
    const int hz = (kz - 1) / 2, hx = (kx - 1) / 2, hy = (ky - 1) / 2;
    const int Lc = p->lc(d);
    const int64_t tree_off = p->tree_offset(Lc);
    std::vector<int> part_idx, part_level, pair_begin{0}, pair_out;
    std::vector<unsigned char> pair_tap;
    // l: level of the tile (of the outputs); the particles in question live on level l - 1
    for (int l = std::min(Lc, apr.level_max); l > apr.level_min; --l) {
        const int zn = apr.z_num[l], xn = apr.x_num[l], yn = apr.y_num[l];
        const int czn = apr.z_num[l - 1], cxn = apr.x_num[l - 1];
        const bool out_tree = (l == Lc) && (l < apr.level_max);
        const bool z_odd = (zn & 1) != 0, x_odd = (xn & 1) != 0, y_odd = (yn & 1) != 0;
        if (!z_odd && !x_odd && !y_odd) continue;
        for (int zc = 0; zc < czn; ++zc)
            for (int xc = 0; xc < cxn; ++xc) {
                const bool row_cut = (2 * zc + 1 >= zn && kz > 1) || 2 * xc + 1 >= xn;
                // 2-D stencils on flat tiles see the z slices of a coarser particle one by one: a missing slice is no cut
                if (!row_cut && !y_odd) continue;
                const uint64_t row = apr.row(l - 1, zc, xc);
                int64_t b = (int64_t)apr.xz_end[row - 1], e = (int64_t)apr.xz_end[row];
                if (b == e) continue;
                if (!row_cut) {                      // only the last particle of the row can stick out in y
                    if (2 * (int)apr.y[e - 1] + 1 < yn) continue;
                    b = e - 1;
                }
                for (int64_t i = b; i < e; ++i) {
                    const int yc = apr.y[i];
                    part_idx.push_back((int)i); part_level.push_back(l);
                    for (int dz = 0; dz < 2; ++dz)
                        for (int dx = 0; dx < 2; ++dx)
                            for (int dy = 0; dy < 2; ++dy) {
                                const int cz = 2 * zc + dz, cx = 2 * xc + dx, cy = 2 * yc + dy;
                                if (cz >= zn || cx >= xn || cy >= yn) continue;
                                for (int t = 0; t < kz * kx * ky; ++t) {
                                    const int sz = t / (kx * ky), sx = (t / ky) % kx, sy = t % ky;
                                    // the output at o reads cell o + (s - h) with tap t
                                    const int oz = cz - (sz - hz), ox = cx - (sx - hx), oy = cy - (sy - hy);
                                    if (oz < 0 || oz >= zn || ox < 0 || ox >= xn || oy < 0 || oy >= yn) continue;
                                    int64_t o = find_in_row(apr, l, oz, ox, oy);
                                    if (o < 0 && out_tree) {
                                        const int64_t tn = find_in_row(tree, l, oz, ox, oy);
                                        if (tn >= 0) o = tn + tree_off;
                                    }
                                    if (o < 0) continue;
                                    pair_out.push_back((int)o); pair_tap.push_back((unsigned char)t);
                                }
                            }
                    pair_begin.push_back((int)pair_out.size());
                }
            }
    }
    FaceLists fl{};
    fl.n_part = (int)part_idx.size();
    if (fl.n_part > 0) {
        auto upload = [&](void** dst, const void* src, size_t bytes) -> int {
            APRNET_HIP_CHECK(hipMalloc(dst, std::max<size_t>(bytes, 16)));
            if (bytes) APRNET_HIP_CHECK(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
            return 0;
        };
        int rc = upload((void**)&fl.d_part_idx, part_idx.data(), part_idx.size() * 4);
        if (!rc) rc = upload((void**)&fl.d_part_level, part_level.data(), part_level.size() * 4);
        if (!rc) rc = upload((void**)&fl.d_pair_begin, pair_begin.data(), pair_begin.size() * 4);
        if (!rc) rc = upload((void**)&fl.d_pair_out, pair_out.data(), pair_out.size() * 4);
        if (!rc) rc = upload((void**)&fl.d_pair_tap, pair_tap.data(), pair_tap.size());
        if (rc) { free_face_lists(fl); return rc; }
    }
    p->faces[key] = fl;
    *out = fl;
    return 0;
}

void free_face_lists(FaceLists& fl) {
    for (void* q : {(void*)fl.d_part_idx, (void*)fl.d_part_level, (void*)fl.d_pair_begin, (void*)fl.d_pair_out, (void*)fl.d_pair_tap})
        if (q) (void)hipFree(q);
    fl = FaceLists{};
}

template <typename T>
__global__ void __launch_bounds__(64)
face_dx_kernel(const FaceLists fl, const T* __restrict__ gy, int64_t ldy, const T* __restrict__ w, int S_exp, int Cout, int Cin,
               int K, int Lc, T* __restrict__ gx, int64_t ldgx) {
    const int pi = blockIdx.x;
    const int pb = fl.d_pair_begin[pi], pe = fl.d_pair_begin[pi + 1];
    const int s = min(S_exp - 1, Lc - fl.d_part_level[pi]);
    const int64_t o = fl.d_part_idx[pi];
    for (int ci = threadIdx.x; ci < Cin; ci += 64) {
        T acc = 0;
        for (int k = pb; k < pe; ++k) {
            const int64_t src = fl.d_pair_out[k];
            const int t = fl.d_pair_tap[k];
            T sum = 0;
            for (int co = 0; co < Cout; ++co)
                sum += w[(((int64_t)s * Cout + co) * Cin + ci) * K + t] * gy[(int64_t)co * ldy + src];
            acc += sum;
        }
        gx[(int64_t)ci * ldgx + o] += acc;
    }
}

// Adds the face terms to gx.  Runs after the main input-gradient kernel on the same stream.
int launch_face_dx(const FaceLists& fl, const float* gy, int64_t ldy, const float* w, int S_exp, int Cout, int Cin, int K, int Lc,
                   float* gx, int64_t ldgx, hipStream_t st) {
    if (fl.n_part == 0) return 0;
    hipLaunchKernelGGL(face_dx_kernel<float>, dim3((unsigned)fl.n_part), dim3(64), 0, st, fl, gy, ldy, w, S_exp, Cout, Cin, K, Lc, gx, ldgx);
    APRNET_LAUNCH_CHECK("face_dx_kernel");
    return 0;
}

}  // namespace aprnet
