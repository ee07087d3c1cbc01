// aprcore — host-side construction of the APR linear-access structure.
//
// The particle-space CNN operators consume an APR only through three arrays per
// access (APR particles and APR tree): level_xz_vec, xz_end_vec, y_vec.  The
// reference obtains them from LibAPR (an un-vendored submodule, absent from
// /root/reference: .gitmodules:4-6); the array semantics are fixed by the call
// sites, e.g. pyapr/aprnet/cuda/src/conv333_gpu.cu:65-67 (row lookup),
// pyapr/aprnet/cuda/src/conv111_gpu.cu:30-31 (per-level contiguous ranges) and
// pyapr/data_containers/src/BindAPR.hpp:72-108 (serialisable state).
//
// This file is an independent builder with its own particle-selection pipeline
// (LibAPR's converter is not available, so which particles it would pick for a
// given image is unknown).  What it guarantees is the structure the operators
// rely on:
//   * levels 1..level_max for particles, 0..level_max-1 for the tree,
//     level_max = ceil(log2(max dim)), grid of level l = ceil(org / 2^(lmax-l));
//   * particles are the leaves of a 2:1-balanced octree (26-neighbourhood), the
//     tree holds every strict ancestor, every tree node has all of its in-image
//     children present as a particle or a tree node;
//   * index order: level-major, then z, then x, then y ascending.
//
// Plain C ABI (ctypes-friendly); OpenMP inside.
#include <cstdint>
#include <cstring>
#include <cmath>
#include <vector>
#include <algorithm>
#include <string>
#include <omp.h>

namespace {

struct Access {
    int level_min = 0, level_max = 0;
    std::vector<int32_t> z_num, x_num, y_num;   // indexable by level, 0..level_max
    std::vector<uint64_t> level_xz_vec;          // [level_max + 2]
    std::vector<uint64_t> xz_end_vec;            // [level_xz_vec[level_max+1]], leading 0
    std::vector<uint16_t> y_vec;
};

struct Apr {
    int org_z = 1, org_x = 1, org_y = 1;
    int level_max = 1;
    Access apr, tree;
};

thread_local std::string g_err;

inline int ceil_shift(int v, int s) { return (int)(((int64_t)v + ((int64_t)1 << s) - 1) >> s); }

int compute_level_max(int z, int x, int y) {
    int m = std::max(z, std::max(x, y));
    int l = 0;
    while ((1 << l) < m) ++l;
    return std::max(l, 1);
}

struct Dims { int z, x, y; size_t size() const { return (size_t)z * x * y; } };

Dims level_dims(const Apr& a, int level) {
    const int s = a.level_max - level;
    return Dims{ceil_shift(a.org_z, s), ceil_shift(a.org_x, s), ceil_shift(a.org_y, s)};
}

void init_access_dims(const Apr& a, Access& acc, int level_min, int level_max) {
    acc.level_min = level_min;
    acc.level_max = level_max;
    acc.z_num.assign(a.level_max + 1, 1);
    acc.x_num.assign(a.level_max + 1, 1);
    acc.y_num.assign(a.level_max + 1, 1);
    for (int l = 0; l <= a.level_max; ++l) {
        Dims d = level_dims(a, l);
        acc.z_num[l] = d.z; acc.x_num[l] = d.x; acc.y_num[l] = d.y;
    }
    // row table offsets: one leading sentinel entry so that row-1 is always valid
    acc.level_xz_vec.assign(level_max + 2, 1);
    uint64_t counter = 1;
    for (int l = 0; l <= level_max; ++l) {
        acc.level_xz_vec[l] = counter;
        if (l >= level_min) counter += (uint64_t)acc.x_num[l] * acc.z_num[l];
    }
    acc.level_xz_vec[level_max + 1] = counter;
    acc.xz_end_vec.assign(counter, 0);
}

// Emit one access (particles or tree) given a per-cell predicate.
template <class Pred>
void emit_access(Access& acc, Pred is_member) {
    const int lmin = acc.level_min, lmax = acc.level_max;
    // pass 1: per-row counts
    for (int l = lmin; l <= lmax; ++l) {
        const int zn = acc.z_num[l], xn = acc.x_num[l], yn = acc.y_num[l];
        const uint64_t base = acc.level_xz_vec[l];
#pragma omp parallel for schedule(dynamic, 4)
        for (int z = 0; z < zn; ++z) {
            for (int x = 0; x < xn; ++x) {
                uint64_t c = 0;
                for (int y = 0; y < yn; ++y) c += is_member(l, z, x, y) ? 1 : 0;
                acc.xz_end_vec[base + (uint64_t)z * xn + x] = c;
            }
        }
    }
    // global inclusive prefix sum (row table is level-major, z, x)
    uint64_t run = 0;
    for (size_t i = 1; i < acc.xz_end_vec.size(); ++i) { run += acc.xz_end_vec[i]; acc.xz_end_vec[i] = run; }
    acc.y_vec.assign(run, 0);
    // pass 2: fill y
    for (int l = lmin; l <= lmax; ++l) {
        const int zn = acc.z_num[l], xn = acc.x_num[l], yn = acc.y_num[l];
        const uint64_t base = acc.level_xz_vec[l];
#pragma omp parallel for schedule(dynamic, 4)
        for (int z = 0; z < zn; ++z) {
            for (int x = 0; x < xn; ++x) {
                const uint64_t row = base + (uint64_t)z * xn + x;
                uint64_t o = acc.xz_end_vec[row - 1];
                if (o == acc.xz_end_vec[row]) continue;
                for (int y = 0; y < yn; ++y) if (is_member(l, z, x, y)) acc.y_vec[o++] = (uint16_t)y;
            }
        }
    }
}

// desired: required level per cell of the level (lmax-1) grid, values 0..lmax
void build_from_desired(Apr& a, const uint8_t* desired) {
    const int lmax = a.level_max;
    std::vector<std::vector<uint8_t>> split(lmax);     // split[l]: node of level l is interior
    std::vector<uint8_t> need, need_prev;
    // pyramid of the maximum required level
    {
        Dims d = level_dims(a, lmax - 1);
        need.assign(desired, desired + d.size());
    }
    for (int l = lmax - 1; l >= 0; --l) {
        Dims d = level_dims(a, l);
        split[l].resize(d.size());
        const uint8_t th = (uint8_t)l;
#pragma omp parallel for
        for (int64_t i = 0; i < (int64_t)d.size(); ++i) split[l][i] = need[i] > th ? 1 : 0;
        if (l == 0) break;
        Dims c = level_dims(a, l - 1);
        need_prev.assign(c.size(), 0);
#pragma omp parallel for
        for (int z = 0; z < c.z; ++z)
            for (int x = 0; x < c.x; ++x)
                for (int y = 0; y < c.y; ++y) {
                    uint8_t m = 0;
                    for (int dz = 0; dz < 2; ++dz) { int zz = 2 * z + dz; if (zz >= d.z) continue;
                    for (int dx = 0; dx < 2; ++dx) { int xx = 2 * x + dx; if (xx >= d.x) continue;
                    for (int dy = 0; dy < 2; ++dy) { int yy = 2 * y + dy; if (yy >= d.y) continue;
                        m = std::max(m, need[((size_t)zz * d.x + xx) * d.y + yy]); }}}
                    need_prev[((size_t)z * c.x + x) * c.y + y] = m;
                }
        need.swap(need_prev);
    }
    std::fill(split[0].begin(), split[0].end(), 1);    // the root is always interior
    // 2:1 balance over the 26-neighbourhood, fine -> coarse: an interior node forces
    // all of its same-level neighbours to exist, i.e. their parents to be interior.
    for (int l = lmax - 1; l >= 1; --l) {
        Dims d = level_dims(a, l), c = level_dims(a, l - 1);
        const std::vector<uint8_t>& s = split[l];
        std::vector<uint8_t>& p = split[l - 1];
#pragma omp parallel for schedule(dynamic, 2)
        for (int z = 0; z < d.z; ++z)
            for (int x = 0; x < d.x; ++x)
                for (int y = 0; y < d.y; ++y) {
                    if (!s[((size_t)z * d.x + x) * d.y + y]) continue;
                    const int z0 = std::max(z - 1, 0) >> 1, z1 = std::min(z + 1, d.z - 1) >> 1;
                    const int x0 = std::max(x - 1, 0) >> 1, x1 = std::min(x + 1, d.x - 1) >> 1;
                    const int y0 = std::max(y - 1, 0) >> 1, y1 = std::min(y + 1, d.y - 1) >> 1;
                    for (int zz = z0; zz <= z1; ++zz)
                        for (int xx = x0; xx <= x1; ++xx)
                            for (int yy = y0; yy <= y1; ++yy) {
                                uint8_t& t = p[((size_t)zz * c.x + xx) * c.y + yy];
                                if (!t) {
#pragma omp atomic write
                                    t = 1;
                                }
                            }
                }
    }
    init_access_dims(a, a.apr, 1, lmax);
    init_access_dims(a, a.tree, 0, lmax - 1);
    auto is_tree = [&](int l, int z, int x, int y) -> bool {
        const int xn = a.tree.x_num[l], yn = a.tree.y_num[l];
        return split[l][((size_t)z * xn + x) * yn + y] != 0;
    };
    auto is_part = [&](int l, int z, int x, int y) -> bool {
        const int pxn = a.apr.x_num[l - 1], pyn = a.apr.y_num[l - 1];
        if (!split[l - 1][((size_t)(z >> 1) * pxn + (x >> 1)) * pyn + (y >> 1)]) return false;
        if (l == lmax) return true;
        return !is_tree(l, z, x, y);
    };
    emit_access(a.apr, is_part);
    emit_access(a.tree, is_tree);
}

// ---------------------------------------------------------------- counter-based RNG
inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
inline double u01(uint64_t h) { return ((h >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
struct Rng {
    uint64_t key, ctr = 0;
    explicit Rng(uint64_t seed) : key(splitmix64(seed ^ 0xA5A5A5A5DEADBEEFull)) {}
    double uniform() { return u01(splitmix64(key + (ctr++) * 0xD1B54A32D192ED03ull)); }
    double uniform(double a, double b) { return a + (b - a) * uniform(); }
};
inline float normal_at(uint64_t seed, uint64_t i) {
    const uint64_t h1 = splitmix64(seed * 0x9E3779B97F4A7C15ull + 2 * i);
    const uint64_t h2 = splitmix64(seed * 0x9E3779B97F4A7C15ull + 2 * i + 1);
    const double u1 = u01(h1), u2 = u01(h2);
    return (float)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
}

struct Blob { float cz, cx, cy, az, ax, ay, amp; };

// separable 1-D filters on a (z, x, y) float volume
void filter_axis(std::vector<float>& v, Dims d, int axis, const float* k, int r) {
    const int n = axis == 0 ? d.z : axis == 1 ? d.x : d.y;
    if (n == 1) return;
    const size_t stride = axis == 0 ? (size_t)d.x * d.y : axis == 1 ? (size_t)d.y : 1;
    const int64_t lines = (int64_t)(d.size() / n);
#pragma omp parallel
    {
        std::vector<float> tmp(n);
#pragma omp for schedule(static)
        for (int64_t line = 0; line < lines; ++line) {
            size_t base;
            if (axis == 2) base = (size_t)line * d.y;
            else if (axis == 1) { size_t z = line / d.y, y = line % d.y; base = z * (size_t)d.x * d.y + y; }
            else base = (size_t)line;
            for (int i = 0; i < n; ++i) {
                float acc = 0;
                for (int t = -r; t <= r; ++t) {
                    int j = std::min(std::max(i + t, 0), n - 1);   // clamp (replicate border)
                    acc += k[t + r] * v[base + j * stride];
                }
                tmp[i] = acc;
            }
            for (int i = 0; i < n; ++i) v[base + i * stride] = tmp[i];
        }
    }
}

}  // namespace

extern "C" {

const char* aprcore_last_error() { return g_err.c_str(); }

void* aprcore_create(int org_z, int org_x, int org_y) {
    if (org_z < 1 || org_x < 1 || org_y < 1 || std::max(org_z, std::max(org_x, org_y)) > 65536) {
        g_err = "aprcore_create: dimensions must be in [1, 65536]"; return nullptr;
    }
    Apr* a = new Apr();
    a->org_z = org_z; a->org_x = org_x; a->org_y = org_y;
    a->level_max = compute_level_max(org_z, org_x, org_y);
    return a;
}

void aprcore_destroy(void* h) { delete static_cast<Apr*>(h); }

int aprcore_level_max(void* h) { return static_cast<Apr*>(h)->level_max; }

// dims of the level-l grid, out = {z, x, y}
void aprcore_level_dims(void* h, int level, int32_t* out) {
    Dims d = level_dims(*static_cast<Apr*>(h), level);
    out[0] = d.z; out[1] = d.x; out[2] = d.y;
}

// desired: uint8 field on the level (level_max-1) grid (C order z,x,y)
int aprcore_build_from_levels(void* h, const uint8_t* desired) {
    build_from_desired(*static_cast<Apr*>(h), desired);
    return 0;
}

// sizes: which = 0 particles, 1 tree; out = {level_min, level_max, n_rows_table, n_particles}
void aprcore_access_info(void* h, int which, int64_t* out) {
    Apr* a = static_cast<Apr*>(h);
    const Access& acc = which ? a->tree : a->apr;
    out[0] = acc.level_min; out[1] = acc.level_max;
    out[2] = (int64_t)acc.xz_end_vec.size(); out[3] = (int64_t)acc.y_vec.size();
}

void aprcore_access_copy(void* h, int which, int32_t* z_num, int32_t* x_num, int32_t* y_num,
                         uint64_t* level_xz_vec, uint64_t* xz_end_vec, uint16_t* y_vec) {
    Apr* a = static_cast<Apr*>(h);
    const Access& acc = which ? a->tree : a->apr;
    const int nl = a->level_max + 1;
    std::memcpy(z_num, acc.z_num.data(), nl * sizeof(int32_t));
    std::memcpy(x_num, acc.x_num.data(), nl * sizeof(int32_t));
    std::memcpy(y_num, acc.y_num.data(), nl * sizeof(int32_t));
    std::memcpy(level_xz_vec, acc.level_xz_vec.data(), acc.level_xz_vec.size() * sizeof(uint64_t));
    std::memcpy(xz_end_vec, acc.xz_end_vec.data(), acc.xz_end_vec.size() * sizeof(uint64_t));
    if (!acc.y_vec.empty()) std::memcpy(y_vec, acc.y_vec.data(), acc.y_vec.size() * sizeof(uint16_t));
}

// ---------------------------------------------------------------- image -> required-level field
// img: uint16 (z, x, y).  out: uint8 on the level (lmax-1) grid.
// Own pipeline in the spirit of pyapr/converter/src/BindConverter.hpp:131-157:
// gradient magnitude and a local intensity scale on the 2x-downsampled grid, thresholds,
// level = min(floor(lmax + log2(|grad| / (sigma * rel_error))), lmax).
int aprcore_level_field_u16(void* h, const uint16_t* img, float rel_error, float smoothing,
                            float ip_th, float sigma_th, float grad_th, uint8_t* out) {
    Apr* a = static_cast<Apr*>(h);
    const int lmax = a->level_max;
    const Dims o{a->org_z, a->org_x, a->org_y};
    const Dims d = level_dims(*a, lmax - 1);
    std::vector<float> g(d.size());
#pragma omp parallel for schedule(static)
    for (int z = 0; z < d.z; ++z)
        for (int x = 0; x < d.x; ++x)
            for (int y = 0; y < d.y; ++y) {
                float s = 0; int c = 0;
                for (int dz = 0; dz < 2; ++dz) { int zz = 2 * z + dz; if (zz >= o.z) continue;
                for (int dx = 0; dx < 2; ++dx) { int xx = 2 * x + dx; if (xx >= o.x) continue;
                for (int dy = 0; dy < 2; ++dy) { int yy = 2 * y + dy; if (yy >= o.y) continue;
                    s += img[((size_t)zz * o.x + xx) * o.y + yy]; ++c; }}}
                g[((size_t)z * d.x + x) * d.y + y] = s / c;
            }
    const float k3[3] = {0.25f, 0.5f, 0.25f};
    const int passes = std::max(0, (int)std::lround(smoothing));
    for (int p = 0; p < passes; ++p) for (int ax = 0; ax < 3; ++ax) filter_axis(g, d, ax, k3, 1);
    // local intensity scale: box-mean of |g - boxmean(g)|, radius 2
    const float k5[5] = {0.2f, 0.2f, 0.2f, 0.2f, 0.2f};
    std::vector<float> m(g);
    for (int ax = 0; ax < 3; ++ax) filter_axis(m, d, ax, k5, 2);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)d.size(); ++i) m[i] = std::fabs(g[i] - m[i]);
    for (int ax = 0; ax < 3; ++ax) filter_axis(m, d, ax, k5, 2);
    const float inv_e = 1.0f / rel_error;
#pragma omp parallel for schedule(static)
    for (int z = 0; z < d.z; ++z)
        for (int x = 0; x < d.x; ++x)
            for (int y = 0; y < d.y; ++y) {
                const size_t i = ((size_t)z * d.x + x) * d.y + y;
                auto at = [&](int zz, int xx, int yy) {
                    zz = std::min(std::max(zz, 0), d.z - 1); xx = std::min(std::max(xx, 0), d.x - 1);
                    yy = std::min(std::max(yy, 0), d.y - 1);
                    return g[((size_t)zz * d.x + xx) * d.y + yy];
                };
                // central differences; the half-resolution grid has a spacing of 2 pixels
                const float gz = d.z > 1 ? (at(z + 1, x, y) - at(z - 1, x, y)) * 0.25f : 0.f;
                const float gx = d.x > 1 ? (at(z, x + 1, y) - at(z, x - 1, y)) * 0.25f : 0.f;
                const float gy = d.y > 1 ? (at(z, x, y + 1) - at(z, x, y - 1)) * 0.25f : 0.f;
                float grad = std::sqrt(gz * gz + gx * gx + gy * gy);
                if (grad < grad_th || g[i] < ip_th) grad = 0.f;
                const float sigma = std::max(m[i], sigma_th);
                int level = 0;
                if (grad > 0.f) {
                    const float L = grad * inv_e / sigma;          // 1 / (admissible cell size in pixels)
                    level = (int)std::floor((float)lmax + std::log2(L));
                    level = std::min(std::max(level, 0), lmax);
                }
                out[i] = (uint8_t)level;
            }
    return 0;
}

// Mean of the image over each particle cell (particle intensities are cell means,
// pyapr/converter/converter_methods.py:36,65).  out: float [n_particles]
int aprcore_sample_mean_u16(void* h, const uint16_t* img, float* out) {
    Apr* a = static_cast<Apr*>(h);
    const Access& acc = a->apr;
    const Dims o{a->org_z, a->org_x, a->org_y};
    for (int l = acc.level_min; l <= acc.level_max; ++l) {
        const int s = a->level_max - l, w = 1 << s;
        const int zn = acc.z_num[l], xn = acc.x_num[l];
        const uint64_t base = acc.level_xz_vec[l];
#pragma omp parallel for schedule(dynamic, 2)
        for (int z = 0; z < zn; ++z)
            for (int x = 0; x < xn; ++x) {
                const uint64_t row = base + (uint64_t)z * xn + x;
                for (uint64_t i = acc.xz_end_vec[row - 1]; i < acc.xz_end_vec[row]; ++i) {
                    const int y = acc.y_vec[i];
                    double sum = 0; int c = 0;
                    for (int zz = z * w; zz < std::min((z + 1) * w, o.z); ++zz)
                        for (int xx = x * w; xx < std::min((x + 1) * w, o.x); ++xx)
                            for (int yy = y * w; yy < std::min((y + 1) * w, o.y); ++yy) {
                                sum += img[((size_t)zz * o.x + xx) * o.y + yy]; ++c;
                            }
                    out[i] = (float)(sum / c);
                }
            }
    }
    return 0;
}

// ---------------------------------------------------------------- seeded synthetic volumes
// kind 0: Gaussian blobs   amp * exp(-0.5 * rho^2), rho^2 = sum ((p-c)/a)^2, a = "sigma" per axis
// kind 1: soft-edged solid ellipsoids, amp inside, one-pixel linear edge
// Blob parameters: semi-axes U[a_lo, a_hi] (isotropic if iso != 0), amplitude U[amp_lo, amp_hi].
// Background: bg_lo + (bg_hi - bg_lo) * low-frequency sinusoid product (constant when equal).
// Noise: Poisson approximated by round(lambda + sqrt(lambda) * N(0,1)) (lambda >= 100 everywhere),
// with N(0,1) a pure function of (seed, voxel index), so the stream never depends on threads.
int aprcore_synth_volume_u16(uint16_t* img, int nz, int nx, int ny, uint64_t seed, int kind,
                             int n_blobs, float a_lo, float a_hi, int iso, float amp_lo, float amp_hi,
                             float bg_lo, float bg_hi, int poisson) {
    std::vector<Blob> blobs(n_blobs);
    Rng rng(seed);
    for (auto& b : blobs) {
        b.cz = (float)rng.uniform(0, nz); b.cx = (float)rng.uniform(0, nx); b.cy = (float)rng.uniform(0, ny);
        b.az = (float)rng.uniform(a_lo, a_hi);
        b.ax = iso ? b.az : (float)rng.uniform(a_lo, a_hi);
        b.ay = iso ? b.az : (float)rng.uniform(a_lo, a_hi);
        b.amp = (float)rng.uniform(amp_lo, amp_hi);
        if (nz == 1) b.cz = 0.f;
    }
    const float ext = kind == 0 ? 4.0f : 1.0f;   // support in units of the semi-axis
    std::vector<std::vector<int>> by_z(nz);
    for (int i = 0; i < n_blobs; ++i) {
        const Blob& b = blobs[i];
        const int z0 = std::max(0, (int)std::floor(b.cz - ext * b.az - 1)), z1 = std::min(nz - 1, (int)std::ceil(b.cz + ext * b.az + 1));
        for (int z = z0; z <= z1; ++z) by_z[z].push_back(i);
    }
    const double tz = 6.283185307179586 / std::max(nz, 2) * 1.5, tx = 6.283185307179586 / std::max(nx, 2) * 2.0,
                 ty = 6.283185307179586 / std::max(ny, 2) * 2.5;
#pragma omp parallel
    {
        std::vector<float> slice((size_t)nx * ny);
#pragma omp for schedule(dynamic, 1)
        for (int z = 0; z < nz; ++z) {
            std::fill(slice.begin(), slice.end(), 0.f);    // blob layer; background added at the end
            for (int bi : by_z[z]) {
                const Blob& b = blobs[bi];
                const float dz = (z + 0.5f - b.cz) / b.az;
                const int x0 = std::max(0, (int)std::floor(b.cx - ext * b.ax - 1)), x1 = std::min(nx - 1, (int)std::ceil(b.cx + ext * b.ax + 1));
                const int y0 = std::max(0, (int)std::floor(b.cy - ext * b.ay - 1)), y1 = std::min(ny - 1, (int)std::ceil(b.cy + ext * b.ay + 1));
                const float amin = std::min(b.az, std::min(b.ax, b.ay));
                for (int x = x0; x <= x1; ++x) {
                    const float dx = (x + 0.5f - b.cx) / b.ax;
                    for (int y = y0; y <= y1; ++y) {
                        const float dy = (y + 0.5f - b.cy) / b.ay;
                        const float r2 = (nz == 1 ? 0.f : dz * dz) + dx * dx + dy * dy;
                        float v;
                        if (kind == 0) v = r2 < ext * ext ? b.amp * std::exp(-0.5f * r2) : 0.f;
                        else { const float t = (1.0f - std::sqrt(r2)) * amin + 0.5f; v = b.amp * std::min(std::max(t, 0.f), 1.f); }
                        float& s = slice[(size_t)x * ny + y];
                        s = kind == 0 ? s + v : std::max(s, v);
                    }
                }
            }
            for (int x = 0; x < nx; ++x)
                for (int y = 0; y < ny; ++y) {
                    const size_t i = ((size_t)z * nx + x) * ny + y;
                    float bg = bg_lo;
                    if (bg_hi > bg_lo) bg = bg_lo + (bg_hi - bg_lo) * (float)(0.5 + 0.5 * std::sin(tz * z) * std::sin(tx * x + 0.7) * std::cos(ty * y));
                    float lam = bg + slice[(size_t)x * ny + y];
                    if (poisson) lam = lam + std::sqrt(std::max(lam, 0.f)) * normal_at(seed, i);
                    img[i] = (uint16_t)std::min(std::max(std::lround(lam), 0l), 65535l);
                }
        }
    }
    return 0;
}

}  // extern "C"
