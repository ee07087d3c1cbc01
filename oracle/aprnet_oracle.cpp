// TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.
//
// CPU restatement (C++17 / OpenMP) of the arithmetic of APR-CNN's CPU operators, written from
// the reference headers under /root/reference/pyapr/aprnet/src (each function cites the lines it
// follows).  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it, and
// only as the checker / the timed CPU baseline.  The shipped operators never call into this file.
//
// The reference headers themselves cannot be compiled here: they include LibAPR headers
// (<data_structures/APR/APR.hpp>, helpers.hpp:10-11) and LibAPR is an empty, un-vendored submodule.
// Only kernel.hpp (RestrictKernel) builds on its own; oracle/ref_restrict.cpp does that.
//
// How each function is pinned (tests/test_oracle_*.py):
//   number_parts / tree_offset   closed form from the row tables
//   parent_index                 brute-force coordinate search
//   fill_tree_mean               avg_pool3d(ceil_mode, count_include_pad=False) on the dense level view
//   conv (all stencils)          F.conv3d on the zero-padded dense level view, sampled at particles
//   conv111                      per-level matmul
//   maxpool (+argmax)            max_pool3d(ceil_mode) + brute-force first-max in traversal order
//   upsample                     nearest-neighbour on the dense view
//   restrict_kernel              the compiled reference (oracle/_ref) + closed-form overlap table
//   reconstruct / sample         dense view; sample(reconstruct(x)) == x (pyapr/tests/test_aprnet.py:272-285)
//   every backward               float64 torch.autograd.gradcheck and <Ax,y> == <x,A'y>
//   particle coords              closed form floor((c + 0.5) * 2^(lmax - l)) through the Python row iterator
//   sample_image (max pyramid)   max_pool3d(ceil_mode) pyramid of the image read at the particles' cells; how LibAPR's
//                                downsamplePyramid treats the far faces of odd-sized images is not visible in the
//                                reference (LibAPR is not vendored): PARITY UNPINNED at those faces
//   labels_to_dist               cuboid labels with axis and diagonal rays (closed-form distances), label 0 and
//                                out-of-image centres left untouched
//
// One deliberate difference: the reference's patch buffer is never cleared, so cells that no source
// covers keep stale values (helpers.hpp:358-420); here every gathered row starts from zero.  On a
// 2:1-balanced APR such cells are never read by a stencil of half-width <= 2, so results agree.
// A second one: backward recomputes the tree means per input channel from a zeroed buffer (the
// reference reuses one buffer across channels, conv.hpp:317-321, which would add channel c-1's
// means to channel c's if the resize does not re-zero).
#include <cstdint>
#include <cstring>
#include <cmath>
#include <vector>
#include <algorithm>
#include <omp.h>

namespace {

struct AccessDesc {               // same layout as aprnet_access_desc (include/aprnet_hip.h)
    int32_t level_min, level_max;
    const int32_t *z_num, *x_num, *y_num;
    const uint64_t* level_xz_vec;
    const uint64_t* xz_end_vec;
    const uint16_t* y_vec;
    uint64_t n_rows, n_particles;
};

struct Acc {
    const AccessDesc& d;
    explicit Acc(const AccessDesc* p) : d(*p) {}
    int lmin() const { return d.level_min; }
    int lmax() const { return d.level_max; }
    int zn(int l) const { return d.z_num[l]; }
    int xn(int l) const { return d.x_num[l]; }
    int yn(int l) const { return d.y_num[l]; }
    uint64_t row(int l, int z, int x) const { return d.level_xz_vec[l] + (uint64_t)z * d.x_num[l] + x; }
    uint64_t beg(int l, int z, int x) const { return d.xz_end_vec[row(l, z, x) - 1]; }
    uint64_t end(int l, int z, int x) const { return d.xz_end_vec[row(l, z, x)]; }
    int y(uint64_t i) const { return d.y_vec[i]; }
    uint64_t level_begin(int l) const { return d.xz_end_vec[d.level_xz_vec[l] - 1]; }
    uint64_t level_end(int l) const { return d.xz_end_vec[d.level_xz_vec[l + 1] - 1]; }
    // cumulative count up to and including level l
    uint64_t total(int l) const { return l < d.level_min ? 0 : level_end(std::min(l, (int)d.level_max)); }
};

// helpers.hpp:113-117
int64_t tree_offset(const Acc& apr, const Acc& tree, int level) {
    const int64_t parts = (int64_t)apr.total(level);
    const int64_t tstart = level <= tree.lmax() ? (int64_t)tree.level_begin(std::max(level, tree.lmin())) : (int64_t)tree.d.n_particles;
    return parts - tstart;
}

// helpers.hpp:86-101
int64_t number_parts(const Acc& apr, const Acc& tree, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
    int64_t n = (int64_t)apr.total(Lc);
    if (Lc <= tree.lmax() && Lc >= tree.lmin()) n += (int64_t)(tree.level_end(Lc) - tree.level_begin(Lc));
    return n;
}

// helpers.hpp:133-153: 1 / (number of children of the parent that lie inside the image)
struct Scale {
    float xz, yxz;
    int last_y;
};
inline Scale child_scale(const Acc& child, const Acc& parent, int level, int z, int x) {
    const int bx = ((2 * parent.xn(level - 1)) != child.xn(level)) && ((x / 2) == parent.xn(level - 1) - 1);
    const int bz = ((2 * parent.zn(level - 1)) != child.zn(level)) && ((z / 2) == parent.zn(level - 1) - 1);
    Scale s;
    s.xz = std::max((float)(bx + bz) * 2.0f, 1.0f) / 8.0f;
    s.yxz = ((2 * parent.yn(level - 1)) != child.yn(level)) ? s.xz * 2.0f : s.xz;
    s.last_y = parent.yn(level - 1) - 1;
    return s;
}

// Visit every (child, parent) pair of one child level: children of `child` access at `level`,
// parents in `tree` at level-1; merge walk of helpers.hpp:185-194.
template <class F>
void for_children(const Acc& child, const Acc& tree, int level, int chunk, F f) {
    const int zn = child.zn(level), xn = child.xn(level);
#pragma omp parallel for schedule(dynamic, chunk)
    for (int z = 0; z < zn; ++z) {
        for (int x = 0; x < xn; ++x) {
            const Scale sc = child_scale(child, tree, level, z, x);
            uint64_t p = tree.beg(level - 1, z / 2, x / 2);
            const uint64_t e = child.end(level, z, x);
            for (uint64_t c = child.beg(level, z, x); c < e; ++c) {
                const int yp = child.y(c) / 2;
                while (tree.y(p) < yp) ++p;
                f(c, p, tree.y(p) == sc.last_y ? sc.yxz : sc.xz);
            }
        }
    }
}

// helpers.hpp:156-252
template <typename T>
void fill_tree_mean(const Acc& apr, const Acc& tree, const T* in, T* td, int Lc) {
    const uint64_t nt = tree.total(Lc - 1);
    std::fill(td, td + nt, T(0));
    if (Lc < apr.lmax()) {
        const int64_t off = tree_offset(apr, tree, Lc);
        for_children(tree, tree, Lc, 2, [&](uint64_t c, uint64_t p, float s) { td[p] += s * in[c + off]; });
    }
    for (int level = Lc; level >= apr.lmin(); --level)
        for_children(apr, tree, level, 2, [&](uint64_t c, uint64_t p, float s) { td[p] += s * in[c]; });
    for (int level = std::min(Lc - 1, tree.lmax()); level > tree.lmin(); --level)
        for_children(tree, tree, level, 2, [&](uint64_t c, uint64_t p, float s) { td[p] += s * td[c]; });
}

// helpers.hpp:255-350
template <typename T>
void fill_tree_mean_backward(const Acc& apr, const Acc& tree, T* gin, T* gt, int Lc) {
    for (int level = tree.lmin() + 1; level <= std::min(Lc - 1, tree.lmax()); ++level)
        for_children(tree, tree, level, 1, [&](uint64_t c, uint64_t p, float s) { gt[c] += s * gt[p]; });
    for (int level = Lc; level >= apr.lmin(); --level)
        for_children(apr, tree, level, 1, [&](uint64_t c, uint64_t p, float s) { gin[c] += s * gt[p]; });
    if (Lc < apr.lmax()) {
        const int64_t off = tree_offset(apr, tree, Lc);
        for_children(tree, tree, Lc, 1, [&](uint64_t c, uint64_t p, float s) { gin[c + off] += s * gt[p]; });
    }
}

// ------------------------------------------------------------------------------------------------
// Isotropic patch: KZ x KX rows of (y_num + KY - 1) cells, y fastest (APRNetImageBuffer.hpp:8-59)
template <typename T>
struct Patch {
    int ypad = 0, kx = 0, kz = 0;
    std::vector<T> m;
    void shape(int ypad_, int kx_, int kz_) { ypad = ypad_; kx = kx_; kz = kz_; m.assign((size_t)ypad * kx * kz, T(0)); }
    T* row(int zs, int xs) { return m.data() + ((size_t)zs * kx + xs) * ypad; }
    const T* row(int zs, int xs) const { return m.data() + ((size_t)zs * kx + xs) * ypad; }
};

// helpers.hpp:358-420 — one sparse row -> dense y line from three sources, zero elsewhere.
// dst is the padded row (cell y lives at dst[y + HY]).
template <typename T, int HY>
void gather_row(const Acc& apr, const Acc& tree, int level, int z, int x, const T* in, const T* td, int Lc,
                T* dst, int ypad) {
    std::fill(dst, dst + ypad, T(0));
    T* c = dst + HY;
    for (uint64_t i = apr.beg(level, z, x), e = apr.end(level, z, x); i < e; ++i) c[apr.y(i)] = in[i];
    if (level > apr.lmin()) {
        const int yn = apr.yn(level);
        for (uint64_t i = apr.beg(level - 1, z / 2, x / 2), e = apr.end(level - 1, z / 2, x / 2); i < e; ++i) {
            const int y0 = 2 * apr.y(i), y1 = std::min(y0 + 2, yn);
            for (int yy = y0; yy < y1; ++yy) c[yy] = in[i];
        }
    }
    if (level < apr.lmax()) {
        if (level == Lc) {
            const int64_t off = tree_offset(apr, tree, level);
            for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) c[tree.y(i)] = in[i + off];
        } else {
            for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) c[tree.y(i)] = td[i];
        }
    }
}

// helpers.hpp:423-478 — transpose of gather_row
template <typename T, int HY>
void scatter_row_backward(const Acc& apr, const Acc& tree, int level, int z, int x, T* gin, T* gt, int Lc,
                          const T* src) {
    const T* c = src + HY;
    for (uint64_t i = apr.beg(level, z, x), e = apr.end(level, z, x); i < e; ++i) gin[i] += c[apr.y(i)];
    if (level > apr.lmin()) {
        const int yn = apr.yn(level);
        for (uint64_t i = apr.beg(level - 1, z / 2, x / 2), e = apr.end(level - 1, z / 2, x / 2); i < e; ++i) {
            const int y0 = 2 * apr.y(i), y1 = std::min(y0 + 2, yn);
            for (int yy = y0; yy < y1; ++yy) gin[i] += c[yy];
        }
    }
    if (level < apr.lmax()) {
        if (level == Lc) {
            const int64_t off = tree_offset(apr, tree, level);
            for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) gin[i + off] += c[tree.y(i)];
        } else {
            for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) gt[i] += c[tree.y(i)];
        }
    }
}

// Visit the output positions of row (level, z, x): particles, plus the downsampled particles
// when level == Lc < level_max (helpers.hpp:521-574).
template <class F>
inline void for_outputs(const Acc& apr, const Acc& tree, int level, int z, int x, int Lc, F f) {
    for (uint64_t i = apr.beg(level, z, x), e = apr.end(level, z, x); i < e; ++i) f(i, apr.y(i));
    if (level < apr.lmax() && level == Lc) {
        const int64_t off = tree_offset(apr, tree, level);
        for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) f(i + off, tree.y(i));
    }
}

// conv.hpp:83-195 with helpers.hpp:505-575.  w: [Cin][S][Cout][KZ*KX*KY].
template <typename T, int KZ, int KX, int KY>
void conv_forward(const Acc& apr, const Acc& tree, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout,
                  T* out, int64_t ldo, int level_delta) {
    constexpr int HZ = (KZ - 1) / 2, HX = (KX - 1) / 2, HY = (KY - 1) / 2, K = KZ * KX * KY;
    const int Lc = apr.lmax() - level_delta;
    std::vector<T> td(std::max<uint64_t>(tree.total(Lc - 1), 1));
    for (int ci = 0; ci < Cin; ++ci) {
        const T* in = x + ci * ldx;
        fill_tree_mean(apr, tree, in, td.data(), Lc);
#pragma omp parallel
        {
            Patch<T> patch;
            T taps[K];
            for (int level = Lc; level >= apr.lmin(); --level) {
                const int s_idx = std::min(S - 1, Lc - level);
                const T* filt = w + ((size_t)ci * S + s_idx) * Cout * K;
                const int zn = apr.zn(level), xn = apr.xn(level), ypad = apr.yn(level) + KY - 1;
#pragma omp for schedule(dynamic)
                for (int z = 0; z < zn; ++z) {
                    patch.shape(ypad, KX, KZ);            // all zero: out-of-grid rows stay zero
                    auto load_col = [&](int xc) {         // column xc of rows z-HZ..z+HZ into slot xc mod KX
                        const int xs = ((xc % KX) + KX) % KX;
                        for (int dz = 0; dz < KZ; ++dz) {
                            const int zz = z - HZ + dz;
                            T* dst = patch.row(dz, xs);
                            if (zz < 0 || zz >= zn || xc < 0 || xc >= xn) std::fill(dst, dst + ypad, T(0));
                            else gather_row<T, HY>(apr, tree, level, zz, xc, in, td.data(), Lc, dst, ypad);
                        }
                    };
                    for (int xc = -HX; xc < HX; ++xc) load_col(xc);
                    for (int xx = 0; xx < xn; ++xx) {
                        load_col(xx + HX);
                        for_outputs(apr, tree, level, z, xx, Lc, [&](uint64_t idx, int y) {
                            int k = 0;
                            for (int sz = 0; sz < KZ; ++sz)
                                for (int sx = 0; sx < KX; ++sx) {
                                    const T* r = patch.row(sz, (((xx - HX + sx) % KX) + KX) % KX) + y;
                                    for (int sy = 0; sy < KY; ++sy) taps[k++] = r[sy];
                                }
                            for (int co = 0; co < Cout; ++co) {
                                const T* wp = filt + (size_t)co * K;
                                T res = 0;
                                for (int i = 0; i < K; ++i) res += taps[i] * wp[i];
                                out[co * ldo + idx] += res;
                            }
                        });
                    }
                }
            }
        }
    }
}

// conv.hpp:289-481 with helpers.hpp:578-704.  gw: [Cin][S][Cout][K], accumulated.
template <typename T, int KZ, int KX, int KY>
void conv_backward(const Acc& apr, const Acc& tree, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout,
                   const T* gout, int64_t ldo, T* gin_all, int64_t ldg, T* gw, int level_delta) {
    constexpr int HZ = (KZ - 1) / 2, HX = (KX - 1) / 2, HY = (KY - 1) / 2, K = KZ * KX * KY;
    const int Lc = apr.lmax() - level_delta;
    const uint64_t nt = std::max<uint64_t>(tree.total(Lc - 1), 1);
    const int64_t np = number_parts(apr, tree, level_delta);
    std::vector<T> td(nt), gt(nt);
    for (int ci = 0; ci < Cin; ++ci) {
        const T* in = x + ci * ldx;
        T* gin = gin_all + ci * ldg;
        fill_tree_mean(apr, tree, in, td.data(), Lc);
        std::fill(gt.begin(), gt.end(), T(0));
#pragma omp parallel
        {
            std::vector<T> gin_loc(np, T(0)), gt_loc(nt, T(0)), dw_loc((size_t)S * Cout * K, T(0));
            T taps[K], gtaps[K];
            std::vector<T> vals, grads;      // slabs [KZ][xn + 2 HX][ypad]
            for (int level = Lc; level >= apr.lmin(); --level) {
                const int s_idx = std::min(S - 1, Lc - level);
                const T* filt = w + ((size_t)ci * S + s_idx) * Cout * K;
                T* dwl = dw_loc.data() + (size_t)s_idx * Cout * K;
                const int zn = apr.zn(level), xn = apr.xn(level), ypad = apr.yn(level) + KY - 1;
                const int xw = xn + 2 * HX;
                auto at = [&](std::vector<T>& v, int dz, int xc) { return v.data() + ((size_t)dz * xw + (xc + HX)) * ypad; };
#pragma omp for schedule(dynamic)
                for (int z = 0; z < zn; ++z) {
                    vals.assign((size_t)KZ * xw * ypad, T(0));
                    grads.assign((size_t)KZ * xw * ypad, T(0));
                    for (int dz = 0; dz < KZ; ++dz) {
                        const int zz = z - HZ + dz;
                        if (zz < 0 || zz >= zn) continue;
                        for (int xc = 0; xc < xn; ++xc)
                            gather_row<T, HY>(apr, tree, level, zz, xc, in, td.data(), Lc, at(vals, dz, xc), ypad);
                    }
                    for (int xx = 0; xx < xn; ++xx) {
                        for_outputs(apr, tree, level, z, xx, Lc, [&](uint64_t idx, int y) {
                            std::fill(gtaps, gtaps + K, T(0));
                            int k = 0;
                            for (int sz = 0; sz < KZ; ++sz)
                                for (int sx = 0; sx < KX; ++sx) {
                                    const T* r = at(vals, sz, xx - HX + sx) + y;
                                    for (int sy = 0; sy < KY; ++sy) taps[k++] = r[sy];
                                }
                            for (int co = 0; co < Cout; ++co) {
                                const T dO = gout[co * ldo + idx];
                                const T* wp = filt + (size_t)co * K;
                                T* dwp = dwl + (size_t)co * K;
                                for (int i = 0; i < K; ++i) { gtaps[i] += dO * wp[i]; dwp[i] += dO * taps[i]; }
                            }
                            k = 0;
                            for (int sz = 0; sz < KZ; ++sz)
                                for (int sx = 0; sx < KX; ++sx) {
                                    T* r = at(grads, sz, xx - HX + sx) + y;
                                    for (int sy = 0; sy < KY; ++sy) r[sy] += gtaps[k++];
                                }
                        });
                    }
                    for (int dz = 0; dz < KZ; ++dz) {
                        const int zz = z - HZ + dz;
                        if (zz < 0 || zz >= zn) continue;
                        for (int xc = 0; xc < xn; ++xc)
                            scatter_row_backward<T, HY>(apr, tree, level, zz, xc, gin_loc.data(), gt_loc.data(), Lc,
                                                        at(grads, dz, xc));
                    }
                }
            }
#pragma omp critical
            {
                for (uint64_t i = 0; i < nt; ++i) gt[i] += gt_loc[i];
                for (int64_t i = 0; i < np; ++i) gin[i] += gin_loc[i];
                T* g = gw + (size_t)ci * S * Cout * K;
                for (size_t i = 0; i < dw_loc.size(); ++i) g[i] += dw_loc[i];
            }
        }
        fill_tree_mean_backward(apr, tree, gin, gt.data(), Lc);
    }
}

// conv.hpp:199-256.  w: [Cin][S][Cout]
template <typename T>
void conv111_forward(const Acc& apr, const Acc& tree, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout,
                     T* out, int64_t ldo, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
#pragma omp parallel for if (Cout > 15)
    for (int co = 0; co < Cout; ++co)
        for (int ci = 0; ci < Cin; ++ci)
            for (int level = Lc; level >= apr.lmin(); --level) {
                const T wv = w[((size_t)ci * S + std::min(S - 1, Lc - level)) * Cout + co];
                const T* in = x + ci * ldx;
                T* o = out + co * ldo;
                for (uint64_t i = apr.level_begin(level), e = apr.level_end(level); i < e; ++i) o[i] = o[i] + wv * in[i];
                if (level == Lc && Lc < apr.lmax()) {
                    const int64_t off = tree_offset(apr, tree, Lc);
                    for (uint64_t i = tree.level_begin(Lc) + off, e = tree.level_end(Lc) + off; i < e; ++i) o[i] = o[i] + wv * in[i];
                }
            }
}

// conv.hpp:484-554
template <typename T>
void conv111_backward(const Acc& apr, const Acc& tree, const T* x, int64_t ldx, int Cin, const T* w, int S, int Cout,
                      const T* gout, int64_t ldo, T* gin_all, int64_t ldg, T* gw, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
#pragma omp parallel for if (Cin > 15)
    for (int ci = 0; ci < Cin; ++ci)
        for (int co = 0; co < Cout; ++co)
            for (int level = Lc; level >= apr.lmin(); --level) {
                const size_t wi = ((size_t)ci * S + std::min(S - 1, Lc - level)) * Cout + co;
                const T wv = w[wi];
                const T* in = x + ci * ldx;
                const T* go = gout + co * ldo;
                T* gi = gin_all + ci * ldg;
                T dw = 0;
                auto span = [&](uint64_t b, uint64_t e) {
                    T acc = 0;
                    for (uint64_t i = b; i < e; ++i) acc = acc + in[i] * go[i];
                    dw += acc;
                    for (uint64_t i = b; i < e; ++i) gi[i] = gi[i] + wv * go[i];
                };
                span(apr.level_begin(level), apr.level_end(level));
                if (level == Lc && Lc < apr.lmax()) {
                    const int64_t off = tree_offset(apr, tree, Lc);
                    span(tree.level_begin(Lc) + off, tree.level_end(Lc) + off);
                }
                gw[wi] += dw;
            }
}

// kernel.hpp:31-126 (forward) / 129-224 (backward).  Tensors [Cin][S or S_exp][Cout][KZ][KX][KY].
template <typename T, bool Backward>
void restrict_kernel(const T* src, T* dst, int Cin, int S, int S_exp, int Cout, int KZ, int KX, int KY) {
    const int ndim = (KZ > 1) + (KX > 1) + (KY > 1);
    const int K = KZ * KX * KY;
    const size_t bank = (size_t)Cout * K;
    auto overlap = [](int o, int i, int off, int step) {
        return std::min((o + 1) * step, off + i + step) - std::max(o * step, off + i);
    };
    for (int ci = 0; ci < Cin; ++ci) {
        const T* s_ci = src + (size_t)ci * (Backward ? S_exp : S) * bank;
        T* d_ci = dst + (size_t)ci * (Backward ? S : S_exp) * bank;
        for (int l = 0; l < S; ++l) std::copy(s_ci + l * bank, s_ci + (l + 1) * bank, d_ci + l * bank);
        for (int l = S; l < S_exp; ++l) {
            const int step = (int)std::pow(2.0f, (float)(l - (S - 1)));
            const float factor = std::pow((float)step, (float)ndim);
            const int zo = (KZ / 2) * step - KZ / 2, xo = (KX / 2) * step - KX / 2, yo = (KY / 2) * step - KY / 2;
            for (int zi = 0; zi < KZ; ++zi) for (int xi = 0; xi < KX; ++xi) for (int yi = 0; yi < KY; ++yi)
            for (int zq = 0; zq < KZ; ++zq) {
                const float oz = (float)overlap(zq, zi, zo, step);
                if (oz <= 0) continue;
                for (int xq = 0; xq < KX; ++xq) {
                    const float ox = (float)std::max(overlap(xq, xi, xo, step), 0);
                    if (ox <= 0) continue;
                    for (int yq = 0; yq < KY; ++yq) {
                        const float oy = (float)std::max(overlap(yq, yi, yo, step), 0);
                        if (oy <= 0) continue;
                        const float ov = ox * oy * oz / factor;
                        const int in_tap = (zi * KX + xi) * KY + yi, out_tap = (zq * KX + xq) * KY + yq;
                        for (int co = 0; co < Cout; ++co) {
                            if (!Backward) d_ci[(size_t)l * bank + co * K + out_tap] += ov * s_ci[(size_t)(S - 1) * bank + co * K + in_tap];
                            else d_ci[(size_t)(S - 1) * bank + co * K + in_tap] += ov * s_ci[(size_t)l * bank + co * K + out_tap];
                        }
                    }
                }
            }
        }
    }
}

// maxpool.hpp:67-146.  out must be pre-filled by the caller (-1e17 in the reference, maxpool.hpp:51).
template <typename T>
void maxpool_forward(const Acc& apr, const Acc& tree, const T* x, int64_t ldx, int C, T* out, int64_t ldo,
                     int64_t* idx, int64_t ldi, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
    const uint64_t ncopy = apr.total(Lc - 1);
    const int64_t ooff = tree_offset(apr, tree, Lc - 1);
    for (int c = 0; c < C; ++c) {
        const T* in = x + c * ldx; T* o = out + c * ldo; int64_t* ix = idx + c * ldi;
        for (uint64_t i = 0; i < ncopy; ++i) o[i] = in[i];
        auto pass = [&](const Acc& child, int64_t ioff) {
            const int zn = child.zn(Lc), xn = child.xn(Lc);
#pragma omp parallel for schedule(dynamic, 2)
            for (int z = 0; z < zn; ++z)
                for (int xx = 0; xx < xn; ++xx) {
                    uint64_t p = tree.beg(Lc - 1, z / 2, xx / 2);
                    for (uint64_t i = child.beg(Lc, z, xx), e = child.end(Lc, z, xx); i < e; ++i) {
                        while (tree.y(p) < child.y(i) / 2) ++p;
                        if (in[i + ioff] > o[p + ooff]) { o[p + ooff] = in[i + ioff]; ix[p + ooff] = (int64_t)i + ioff; }
                    }
                }
        };
        pass(apr, 0);
        if (Lc < apr.lmax()) pass(tree, tree_offset(apr, tree, Lc));
    }
}

// maxpool.hpp:170-230
template <typename T>
void maxpool_backward(const Acc& apr, const Acc& tree, const T* gout, int64_t ldo, int C, T* gin, int64_t ldg,
                      const int64_t* idx, int64_t ldi, int level_delta) {
    const uint64_t nfixed = apr.total(apr.lmax() - level_delta - 1);
    const uint64_t ntotal = (uint64_t)number_parts(apr, tree, level_delta + 1);
    for (int c = 0; c < C; ++c) {
        for (uint64_t i = 0; i < nfixed; ++i) gin[c * ldg + i] = gout[c * ldo + i];
        for (uint64_t i = nfixed; i < ntotal; ++i) gin[c * ldg + idx[c * ldi + i]] = gout[c * ldo + i];
    }
}

// upsample.hpp:72-141 (forward) / 165-236 (backward)
template <typename T, bool Backward>
void upsample(const Acc& apr, const Acc& tree, const T* src, int64_t lds, int C, T* dst, int64_t ldd, int level_delta) {
    const int Li = apr.lmax() - level_delta, Lo = Li + 1;
    const uint64_t ncopy = apr.total(Li);
    const int64_t ioff = tree_offset(apr, tree, Li), ooff = tree_offset(apr, tree, Lo);
    for (int c = 0; c < C; ++c) {
        const T* s = src + c * lds; T* d = dst + c * ldd;
        for (uint64_t i = 0; i < ncopy; ++i) d[i] = s[i];
        auto pass = [&](const Acc& child, int64_t coff) {
            const int zn = child.zn(Lo), xn = child.xn(Lo);
#pragma omp parallel for schedule(dynamic, 2)
            for (int z = 0; z < zn; ++z)
                for (int xx = 0; xx < xn; ++xx) {
                    uint64_t p = tree.beg(Li, z / 2, xx / 2);
                    for (uint64_t i = child.beg(Lo, z, xx), e = child.end(Lo, z, xx); i < e; ++i) {
                        while (tree.y(p) < child.y(i) / 2) ++p;
                        if (!Backward) d[i + coff] = s[p + ioff];
                        else d[p + ioff] += s[i + coff];
                    }
                }
        };
        pass(apr, 0);
        if (Lo <= tree.lmax()) pass(tree, ooff);
    }
}

// cuda/src/reconstruct_gpu.cu:3-127 restated on the CPU (there is no CPU version in the reference).
// img: [C][zn(Lc)][xn(Lc)][yn(Lc)]
template <typename T, bool Backward>
void reconstruct(const Acc& apr, const Acc& tree, T* parts, int64_t ldp, int C, T* img, int64_t ldi, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
    const int zn = apr.zn(Lc), xn = apr.xn(Lc), yn = apr.yn(Lc);
    const int64_t toff = tree_offset(apr, tree, Lc);
    for (int c = 0; c < C; ++c) {
        T* p = parts + c * ldp; T* im = img + c * ldi;
        for (int level = Lc; level >= apr.lmin(); --level) {
            const int f = 1 << (Lc - level);
            for (int z = 0; z < zn; ++z) for (int x = 0; x < xn; ++x) {
                T* line = im + ((size_t)z * xn + x) * yn;
                const int zl = z / f, xl = x / f;
                for (uint64_t i = apr.beg(level, zl, xl), e = apr.end(level, zl, xl); i < e; ++i) {
                    const int y0 = apr.y(i) * f, y1 = std::min(y0 + f, yn);
                    for (int y = y0; y < y1; ++y) { if (!Backward) line[y] = p[i]; else p[i] += line[y]; }
                }
                if (level == Lc && level_delta > 0)
                    for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) {
                        if (!Backward) line[tree.y(i)] = p[i + toff]; else p[i + toff] += line[tree.y(i)];
                    }
            }
        }
    }
}

// cuda/src/sample_particles_gpu.cu:3-145 restated on the CPU: cell mean of the dense image.
template <typename T, bool Backward>
void sample_particles(const Acc& apr, const Acc& tree, T* parts, int64_t ldp, int C, T* img, int64_t ldi, int level_delta) {
    const int Lc = apr.lmax() - level_delta;
    const int zn = apr.zn(Lc), xn = apr.xn(Lc), yn = apr.yn(Lc);
    const int64_t toff = tree_offset(apr, tree, Lc);
    for (int c = 0; c < C; ++c) {
        T* p = parts + c * ldp; T* im = img + c * ldi;
        for (int level = Lc; level >= apr.lmin(); --level) {
            const int f = 1 << (Lc - level);
            const int xnl = (xn + f - 1) / f, znl = (zn + f - 1) / f;
            for (int z = 0; z < zn; ++z) for (int x = 0; x < xn; ++x) {
                T* line = im + ((size_t)z * xn + x) * yn;
                const int zl = z / f, xl = x / f;
                const int xd = xl < xnl - 1 ? f : xn - xl * f, zd = zl < znl - 1 ? f : zn - zl * f;
                for (uint64_t i = apr.beg(level, zl, xl), e = apr.end(level, zl, xl); i < e; ++i) {
                    const int y0 = apr.y(i) * f, y1 = std::min(y0 + f, yn);
                    const T denom = (T)(xd * zd * (y1 - y0));
                    if (!Backward) { T v = 0; for (int y = y0; y < y1; ++y) v += line[y]; p[i] += v / denom; }
                    else { const T v = p[i] / denom; for (int y = y0; y < y1; ++y) line[y] = v; }
                }
                if (level == Lc && level_delta > 0)
                    for (uint64_t i = tree.beg(level, z, x), e = tree.end(level, z, x); i < e; ++i) {
                        if (!Backward) p[i + toff] = line[tree.y(i)]; else line[tree.y(i)] = p[i + toff];
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------- StarDist utilities
// Visits the feature positions at level delta d: particles of levels <= Lc (index = particle index), then the tree
// nodes of level Lc behind them (utils.hpp:100-104, 170-176).  f(level, z, x, y, feature index).
template <typename F>
void for_each_feature(const Acc& apr, const Acc& tree, int d, F f) {
    const int Lc = apr.lmax() - d;
    for (int l = apr.lmin(); l <= Lc; ++l)
        for (int z = 0; z < apr.zn(l); ++z)
            for (int x = 0; x < apr.xn(l); ++x)
                for (uint64_t i = apr.beg(l, z, x); i < apr.end(l, z, x); ++i) f(l, z, x, apr.y(i), (int64_t)i);
    if (d > 0) {
        const int64_t off = tree_offset(apr, tree, Lc);
        for (int z = 0; z < tree.zn(Lc); ++z)
            for (int x = 0; x < tree.xn(Lc); ++x)
                for (uint64_t i = tree.beg(Lc, z, x); i < tree.end(Lc, z, x); ++i) f(Lc, z, x, tree.y(i), (int64_t)i + off);
    }
}

// get_particle_coords, utils.hpp:222-267
void particle_coords(const Acc& apr, const Acc& tree, int d, float* coords) {
    const int lmax = apr.lmax();
    for_each_feature(apr, tree, d, [&](int l, int z, int x, int y, int64_t i) {
        const double s = std::pow(2.0, lmax - l);
        coords[3 * i + 0] = (float)std::floor((z + 0.5) * s);
        coords[3 * i + 1] = (float)std::floor((x + 0.5) * s);
        coords[3 * i + 2] = (float)std::floor((y + 0.5) * s);
    });
}

// sample_image, utils.hpp:270-333: pyramid by maxima, every feature reads the pyramid entry of its cell
void sample_image_max(const Acc& apr, const Acc& tree, int d, const float* img, int zn, int xn, int yn, float* parts) {
    const int lmax = apr.lmax();
    for_each_feature(apr, tree, d, [&](int l, int z, int x, int y, int64_t i) {
        const int f = 1 << (lmax - l);
        float m = -INFINITY;
        bool any = false;
        for (int zz = z * f; zz < std::min((z + 1) * f, zn); ++zz)
            for (int xx = x * f; xx < std::min((x + 1) * f, xn); ++xx)
                for (int yy = y * f; yy < std::min((y + 1) * f, yn); ++yy) { m = std::max(m, img[((int64_t)zz * xn + xx) * yn + yy]); any = true; }
        parts[i] = any ? m : 0.f;
    });
}

// labels_to_dist_cpp, utils.hpp:86-219
template <typename L>
void labels_to_dist(const Acc& apr, const Acc& tree, int d, const L* img, int zn, int xn, int yn, const float* dzs,
                    const float* dxs, const float* dys, int n_rays, int max_steps, float* dist) {
    const int lmax = apr.lmax();
    for_each_feature(apr, tree, d, [&](int l, int z, int x, int y, int64_t idx) {
        const double s = std::pow(2.0, lmax - l);
        const int i = (int)std::floor((z + 0.5) * s), j = (int)std::floor((x + 0.5) * s), k = (int)std::floor((y + 0.5) * s);
        if (i >= zn || j >= xn || k >= yn) return;
        const L value = img[((int64_t)i * xn + j) * yn + k];
        if (value == 0) return;
        for (int n = 0; n < n_rays; ++n) {
            float xx = 0.f, yy = 0.f, zz = 0.f;
            const float dz = dzs[n], dx = dxs[n], dy = dys[n];
            for (int step = 0; step < max_steps; ++step) {
                xx += dx; yy += dy; zz += dz;
                const long ii = std::lrint((float)i + zz), jj = std::lrint((float)j + xx), kk = std::lrint((float)k + yy);
                if (ii < 0 || ii >= zn || jj < 0 || jj >= xn || kk < 0 || kk >= yn || value != img[((int64_t)ii * xn + jj) * yn + kk])
                    break;
            }
            zz = (float)std::lrint(zz); xx = (float)std::lrint(xx); yy = (float)std::lrint(yy);
            dist[idx * n_rays + n] = std::sqrt(xx * xx + yy * yy + zz * zz);
        }
    });
}

template <typename T>
int conv_fwd_dispatch(int kz, int kx, int ky, const Acc& a, const Acc& t, const T* x, int64_t ldx, int Cin, const T* w,
                      int S, int Cout, T* out, int64_t ldo, int d) {
    const int code = kz * 100 + kx * 10 + ky;
    switch (code) {
        case 333: conv_forward<T, 3, 3, 3>(a, t, x, ldx, Cin, w, S, Cout, out, ldo, d); return 0;
        case 133: conv_forward<T, 1, 3, 3>(a, t, x, ldx, Cin, w, S, Cout, out, ldo, d); return 0;
        case 155: conv_forward<T, 1, 5, 5>(a, t, x, ldx, Cin, w, S, Cout, out, ldo, d); return 0;
        case 555: conv_forward<T, 5, 5, 5>(a, t, x, ldx, Cin, w, S, Cout, out, ldo, d); return 0;
        case 111: conv111_forward<T>(a, t, x, ldx, Cin, w, S, Cout, out, ldo, d); return 0;
    }
    return -1;
}
template <typename T>
int conv_bwd_dispatch(int kz, int kx, int ky, const Acc& a, const Acc& t, const T* x, int64_t ldx, int Cin, const T* w,
                      int S, int Cout, const T* go, int64_t ldo, T* gi, int64_t ldg, T* gw, int d) {
    const int code = kz * 100 + kx * 10 + ky;
    switch (code) {
        case 333: conv_backward<T, 3, 3, 3>(a, t, x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); return 0;
        case 133: conv_backward<T, 1, 3, 3>(a, t, x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); return 0;
        case 155: conv_backward<T, 1, 5, 5>(a, t, x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); return 0;
        case 555: conv_backward<T, 5, 5, 5>(a, t, x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); return 0;
        case 111: conv111_backward<T>(a, t, x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); return 0;
    }
    return -1;
}

}  // namespace

extern "C" {

// thread count of the OpenMP regions (the CPU baseline is timed with one thread and with all cores)
int oracle_set_threads(int n) { const int before = omp_get_max_threads(); if (n > 0) omp_set_num_threads(n); return before; }

int64_t oracle_number_parts(const AccessDesc* a, const AccessDesc* t, int d) { return number_parts(Acc(a), Acc(t), d); }
int64_t oracle_tree_offset(const AccessDesc* a, const AccessDesc* t, int level) { return tree_offset(Acc(a), Acc(t), level); }

// parent tree index of every child of `level` (which = 0: particles, 1: tree nodes) found by the
// reference's merge walk; out indexed by child index (global within its access)
void oracle_parent_index(const AccessDesc* a, const AccessDesc* t, int which, int level, int64_t* out) {
    Acc apr(a), tree(t);
    const Acc& child = which ? tree : apr;
    for_children(child, tree, level, 2, [&](uint64_t c, uint64_t p, float) { out[c] = (int64_t)p; });
}

#define ORACLE_EXPORT(T, SFX)                                                                                          \
    void oracle_fill_tree_mean_##SFX(const AccessDesc* a, const AccessDesc* t, const T* in, T* td, int d) {            \
        Acc apr(a), tree(t); fill_tree_mean<T>(apr, tree, in, td, apr.lmax() - d); }                                   \
    void oracle_fill_tree_mean_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, T* gin, T* gt, int d) {             \
        Acc apr(a), tree(t); fill_tree_mean_backward<T>(apr, tree, gin, gt, apr.lmax() - d); }                         \
    int oracle_conv_fwd_##SFX(const AccessDesc* a, const AccessDesc* t, int kz, int kx, int ky, const T* x, int64_t ldx,\
                              int Cin, const T* w, int S, int Cout, T* out, int64_t ldo, int d) {                      \
        return conv_fwd_dispatch<T>(kz, kx, ky, Acc(a), Acc(t), x, ldx, Cin, w, S, Cout, out, ldo, d); }               \
    int oracle_conv_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, int kz, int kx, int ky, const T* x, int64_t ldx,\
                              int Cin, const T* w, int S, int Cout, const T* go, int64_t ldo, T* gi, int64_t ldg,      \
                              T* gw, int d) {                                                                          \
        return conv_bwd_dispatch<T>(kz, kx, ky, Acc(a), Acc(t), x, ldx, Cin, w, S, Cout, go, ldo, gi, ldg, gw, d); }   \
    void oracle_restrict_fwd_##SFX(const T* w, T* we, int Cin, int S, int S_exp, int Cout, int kz, int kx, int ky) {   \
        restrict_kernel<T, false>(w, we, Cin, S, S_exp, Cout, kz, kx, ky); }                                           \
    void oracle_restrict_bwd_##SFX(const T* gwe, T* gw, int Cin, int S, int S_exp, int Cout, int kz, int kx, int ky) { \
        restrict_kernel<T, true>(gwe, gw, Cin, S, S_exp, Cout, kz, kx, ky); }                                          \
    void oracle_maxpool_fwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* x, int64_t ldx, int C, T* out,    \
                                  int64_t ldo, int64_t* idx, int64_t ldi, int d) {                                     \
        maxpool_forward<T>(Acc(a), Acc(t), x, ldx, C, out, ldo, idx, ldi, d); }                                        \
    void oracle_maxpool_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* go, int64_t ldo, int C, T* gi,    \
                                  int64_t ldg, const int64_t* idx, int64_t ldi, int d) {                               \
        maxpool_backward<T>(Acc(a), Acc(t), go, ldo, C, gi, ldg, idx, ldi, d); }                                       \
    void oracle_upsample_fwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* x, int64_t ldx, int C, T* out,   \
                                   int64_t ldo, int d) { upsample<T, false>(Acc(a), Acc(t), x, ldx, C, out, ldo, d); } \
    void oracle_upsample_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* go, int64_t ldo, int C, T* gi,   \
                                   int64_t ldg, int d) { upsample<T, true>(Acc(a), Acc(t), go, ldo, C, gi, ldg, d); }  \
    void oracle_reconstruct_fwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* p, int64_t ldp, int C, T* img,\
                                      int64_t ldi, int d) {                                                            \
        reconstruct<T, false>(Acc(a), Acc(t), const_cast<T*>(p), ldp, C, img, ldi, d); }                               \
    void oracle_reconstruct_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, T* gp, int64_t ldp, int C,             \
                                      const T* gimg, int64_t ldi, int d) {                                             \
        reconstruct<T, true>(Acc(a), Acc(t), gp, ldp, C, const_cast<T*>(gimg), ldi, d); }                              \
    void oracle_sample_fwd_##SFX(const AccessDesc* a, const AccessDesc* t, T* p, int64_t ldp, int C, const T* img,     \
                                 int64_t ldi, int d) {                                                                 \
        sample_particles<T, false>(Acc(a), Acc(t), p, ldp, C, const_cast<T*>(img), ldi, d); }                          \
    void oracle_sample_bwd_##SFX(const AccessDesc* a, const AccessDesc* t, const T* gp, int64_t ldp, int C, T* gimg,   \
                                 int64_t ldi, int d) {                                                                 \
        sample_particles<T, true>(Acc(a), Acc(t), const_cast<T*>(gp), ldp, C, gimg, ldi, d); }

ORACLE_EXPORT(float, f32)
ORACLE_EXPORT(double, f64)

void oracle_particle_coords(const AccessDesc* a, const AccessDesc* t, int d, float* coords) { particle_coords(Acc(a), Acc(t), d, coords); }
void oracle_sample_image_max(const AccessDesc* a, const AccessDesc* t, int d, const float* img, int zn, int xn, int yn, float* parts) {
    sample_image_max(Acc(a), Acc(t), d, img, zn, xn, yn, parts);
}
#define ORACLE_LABELS(T, SFX)                                                                                          \
    void oracle_labels_to_dist_##SFX(const AccessDesc* a, const AccessDesc* t, int d, const T* img, int zn, int xn, int yn, \
                                     const float* dzs, const float* dxs, const float* dys, int n_rays, int max_steps,  \
                                     float* dist) {                                                                    \
        labels_to_dist<T>(Acc(a), Acc(t), d, img, zn, xn, yn, dzs, dxs, dys, n_rays, max_steps, dist); }
ORACLE_LABELS(uint8_t, u8)
ORACLE_LABELS(uint16_t, u16)
ORACLE_LABELS(uint32_t, u32)
ORACLE_LABELS(uint64_t, u64)

}  // extern "C"
