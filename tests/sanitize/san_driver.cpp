// Host-only driver for sanitizer builds (AddressSanitizer + UndefinedBehaviorSanitizer) of the two CPU libraries:
// the APR builder (apr-cnn_amd/csrc/aprcore.cpp) and the oracle (oracle/aprnet_oracle.cpp).  It is compiled TOGETHER
// with those two sources into one instrumented executable (tests/test_sanitizers.py), builds an APR of an odd-sized
// synthetic volume and runs every operator of the oracle on it once, forward and backward, at two level deltas.
// Any out-of-bounds access, use after free, leak, signed overflow or misaligned access ends the run with a report.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/aprnet_hip.h"

typedef aprnet_access_desc Desc;
extern "C" {
void* aprcore_create(int, int, int);
void aprcore_destroy(void*);
int aprcore_level_max(void*);
void aprcore_level_dims(void*, int, int32_t*);
int aprcore_build_from_levels(void*, const uint8_t*);
void aprcore_access_info(void*, int, int64_t*);
void aprcore_access_copy(void*, int, int32_t*, int32_t*, int32_t*, uint64_t*, uint64_t*, uint16_t*);
int aprcore_level_field_u16(void*, const uint16_t*, float, float, float, float, float, uint8_t*);
int aprcore_sample_mean_u16(void*, const uint16_t*, float*);
int aprcore_synth_volume_u16(uint16_t*, int, int, int, uint64_t, int, int, float, float, int, float, float, float, float, int);

int64_t oracle_number_parts(const Desc*, const Desc*, int);
int64_t oracle_tree_offset(const Desc*, const Desc*, int);
void oracle_parent_index(const Desc*, const Desc*, int, int, int64_t*);
void oracle_fill_tree_mean_f32(const Desc*, const Desc*, const float*, float*, int);
void oracle_fill_tree_mean_bwd_f32(const Desc*, const Desc*, float*, float*, int);
int oracle_conv_fwd_f32(const Desc*, const Desc*, int, int, int, const float*, int64_t, int, const float*, int, int, float*, int64_t, int);
int oracle_conv_bwd_f32(const Desc*, const Desc*, int, int, int, const float*, int64_t, int, const float*, int, int, const float*, int64_t,
                        float*, int64_t, float*, int);
int oracle_conv_fwd_f64(const Desc*, const Desc*, int, int, int, const double*, int64_t, int, const double*, int, int, double*, int64_t, int);
void oracle_restrict_fwd_f32(const float*, float*, int, int, int, int, int, int, int);
void oracle_restrict_bwd_f32(const float*, float*, int, int, int, int, int, int, int);
void oracle_maxpool_fwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, int64_t*, int64_t, int);
void oracle_maxpool_bwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, const int64_t*, int64_t, int);
void oracle_upsample_fwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, int);
void oracle_upsample_bwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, int);
void oracle_reconstruct_fwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, int);
void oracle_reconstruct_bwd_f32(const Desc*, const Desc*, float*, int64_t, int, const float*, int64_t, int);
void oracle_sample_fwd_f32(const Desc*, const Desc*, float*, int64_t, int, const float*, int64_t, int);
void oracle_sample_bwd_f32(const Desc*, const Desc*, const float*, int64_t, int, float*, int64_t, int);
void oracle_particle_coords(const Desc*, const Desc*, int, float*);
void oracle_sample_image_max(const Desc*, const Desc*, int, const float*, int, int, int, float*);
void oracle_labels_to_dist_u16(const Desc*, const Desc*, int, const uint16_t*, int, int, int, const float*, const float*, const float*, int,
                               int, float*);
}

struct Access {
    std::vector<int32_t> z, x, y;
    std::vector<uint64_t> lxz, xz_end;
    std::vector<uint16_t> yv;
    Desc d{};
    void load(void* h, int which, int apr_level_max) {
        int64_t info[4];
        aprcore_access_info(h, which, info);
        z.resize(apr_level_max + 1); x.resize(apr_level_max + 1); y.resize(apr_level_max + 1);
        lxz.resize((size_t)info[1] + 2); xz_end.resize((size_t)info[2]); yv.resize((size_t)info[3]);
        aprcore_access_copy(h, which, z.data(), x.data(), y.data(), lxz.data(), xz_end.data(), yv.data());
        d.level_min = (int32_t)info[0]; d.level_max = (int32_t)info[1];
        d.z_num = z.data(); d.x_num = x.data(); d.y_num = y.data();
        d.level_xz_vec = lxz.data(); d.xz_end_vec = xz_end.data(); d.y_vec = yv.empty() ? nullptr : yv.data();
        d.n_rows = xz_end.size(); d.n_particles = yv.size();
    }
};

static uint32_t g_state = 12345u;
static float rnd() { g_state = g_state * 1664525u + 1013904223u; return (float)(g_state >> 8) / 16777216.0f - 0.5f; }
static std::vector<float> randv(size_t n) { std::vector<float> v(n); for (auto& e : v) e = rnd(); return v; }
static void check(const std::vector<float>& v, const char* what) {
    for (float e : v) if (!std::isfinite(e)) { std::printf("non-finite value in %s\n", what); std::exit(2); }
}

int main() {
    const int nz = 37, nx = 45, ny = 53;           // odd sizes: far faces cut the coarser cells
    std::vector<uint16_t> img((size_t)nz * nx * ny);
    if (aprcore_synth_volume_u16(img.data(), nz, nx, ny, 7, 0, 12, 2.f, 6.f, 0, 500.f, 2000.f, 90.f, 110.f, 1)) return 3;
    void* h = aprcore_create(nz, nx, ny);
    if (!h) return 3;
    const int lmax = aprcore_level_max(h);
    int32_t dims[3];
    aprcore_level_dims(h, lmax - 1, dims);
    std::vector<uint8_t> field((size_t)dims[0] * dims[1] * dims[2]);
    if (aprcore_level_field_u16(h, img.data(), 0.1f, 1.f, 10.f, 5.f, 3.f, field.data())) return 3;
    if (aprcore_build_from_levels(h, field.data())) return 3;
    Access apr, tree;
    apr.load(h, 0, lmax); tree.load(h, 1, lmax);
    const int64_t n0 = oracle_number_parts(&apr.d, &tree.d, 0), n1 = oracle_number_parts(&apr.d, &tree.d, 1);
    std::printf("particles %lld (level delta 1: %lld), tree nodes %llu, level_max %d\n", (long long)n0, (long long)n1,
                (unsigned long long)tree.d.n_particles, lmax);
    if (n0 <= 0 || n1 <= 0 || (uint64_t)n0 != apr.d.n_particles) return 4;
    std::vector<float> mean((size_t)n0);
    if (aprcore_sample_mean_u16(h, img.data(), mean.data())) return 3;
    check(mean, "sample_mean");
    (void)oracle_tree_offset(&apr.d, &tree.d, lmax - 1);
    std::vector<int64_t> parent(apr.d.n_particles, -1);
    oracle_parent_index(&apr.d, &tree.d, 0, lmax, parent.data());

    const int Cin = 2, Cout = 3, S = 2;
    for (int d = 0; d < 2; ++d) {
        const int64_t n = oracle_number_parts(&apr.d, &tree.d, d);
        const std::vector<float> x = randv((size_t)Cin * n);
        std::vector<float> td((size_t)tree.d.n_particles + 1), gx((size_t)n, 0.f), gt((size_t)tree.d.n_particles + 1, 1.f);
        oracle_fill_tree_mean_f32(&apr.d, &tree.d, x.data(), td.data(), d);
        oracle_fill_tree_mean_bwd_f32(&apr.d, &tree.d, gx.data(), gt.data(), d);
        check(td, "fill_tree_mean"); check(gx, "fill_tree_mean_bwd");
        const int stencils[5][3] = {{3, 3, 3}, {1, 3, 3}, {1, 5, 5}, {5, 5, 5}, {1, 1, 1}};
        for (const auto& k : stencils) {
            const int K = k[0] * k[1] * k[2];
            const std::vector<float> w = randv((size_t)Cin * S * Cout * K), go = randv((size_t)Cout * n);
            std::vector<float> out((size_t)Cout * n, 0.f), gi((size_t)Cin * n, 0.f), gw(w.size(), 0.f);
            if (oracle_conv_fwd_f32(&apr.d, &tree.d, k[0], k[1], k[2], x.data(), n, Cin, w.data(), S, Cout, out.data(), n, d)) return 5;
            if (oracle_conv_bwd_f32(&apr.d, &tree.d, k[0], k[1], k[2], x.data(), n, Cin, w.data(), S, Cout, go.data(), n, gi.data(), n,
                                    gw.data(), d)) return 5;
            check(out, "conv_fwd"); check(gi, "conv_bwd gx"); check(gw, "conv_bwd gw");
        }
        {   // fp64 instantiation of the stencil walk
            std::vector<double> xd(x.begin(), x.end()), wd((size_t)Cin * S * Cout * 27, 0.01), od((size_t)Cout * n, 0.0);
            if (oracle_conv_fwd_f64(&apr.d, &tree.d, 3, 3, 3, xd.data(), n, Cin, wd.data(), S, Cout, od.data(), n, d)) return 5;
        }
        const int64_t np = oracle_number_parts(&apr.d, &tree.d, d + 1);
        std::vector<float> pooled((size_t)Cin * np), gpo = randv((size_t)Cin * np), gpi((size_t)Cin * n, 0.f);
        std::vector<int64_t> arg((size_t)Cin * np);
        oracle_maxpool_fwd_f32(&apr.d, &tree.d, x.data(), n, Cin, pooled.data(), np, arg.data(), np, d);
        oracle_maxpool_bwd_f32(&apr.d, &tree.d, gpo.data(), np, Cin, gpi.data(), n, arg.data(), np, d);
        for (int64_t a : arg) if (a < 0 || a >= n) { std::printf("argmax out of range\n"); return 6; }
        std::vector<float> up((size_t)Cin * n), gup((size_t)Cin * np, 0.f);
        oracle_upsample_fwd_f32(&apr.d, &tree.d, pooled.data(), np, Cin, up.data(), n, d + 1);
        oracle_upsample_bwd_f32(&apr.d, &tree.d, x.data(), n, Cin, gup.data(), np, d + 1);
        check(pooled, "maxpool"); check(gpi, "maxpool_bwd"); check(up, "upsample"); check(gup, "upsample_bwd");
        // dense image at this level delta: dimensions of level lmax - d
        aprcore_level_dims(h, lmax - d, dims);
        const int64_t npix = (int64_t)dims[0] * dims[1] * dims[2];
        std::vector<float> dense((size_t)Cin * npix, 0.f), back((size_t)Cin * n, 0.f), gdense = randv((size_t)Cin * npix), gp((size_t)Cin * n, 0.f);
        oracle_reconstruct_fwd_f32(&apr.d, &tree.d, x.data(), n, Cin, dense.data(), npix, d);
        oracle_sample_fwd_f32(&apr.d, &tree.d, back.data(), n, Cin, dense.data(), npix, d);
        oracle_reconstruct_bwd_f32(&apr.d, &tree.d, gp.data(), n, Cin, gdense.data(), npix, d);
        std::vector<float> gimg((size_t)Cin * npix, 0.f);
        oracle_sample_bwd_f32(&apr.d, &tree.d, x.data(), n, Cin, gimg.data(), npix, d);
        for (size_t i = 0; i < back.size(); ++i)
            if (std::fabs(back[i] - x[i]) > 1e-5f) { std::printf("sample(reconstruct(x)) != x at %zu\n", i); return 7; }
        check(gp, "reconstruct_bwd"); check(gimg, "sample_bwd");
        std::vector<float> coords((size_t)n * 3);
        oracle_particle_coords(&apr.d, &tree.d, d, coords.data());
        check(coords, "particle_coords");
    }
    {   // weight restriction: 3 stencils onto 5 levels and back
        const int K = 27, Sx = 5;
        const std::vector<float> w = randv((size_t)Cin * 3 * Cout * K);
        std::vector<float> we((size_t)Cin * Sx * Cout * K, 0.f), gw(w.size(), 0.f);
        oracle_restrict_fwd_f32(w.data(), we.data(), Cin, 3, Sx, Cout, 3, 3, 3);
        oracle_restrict_bwd_f32(we.data(), gw.data(), Cin, 3, Sx, Cout, 3, 3, 3);
        check(we, "restrict_fwd"); check(gw, "restrict_bwd");
    }
    {   // StarDist utilities on the full-resolution image
        std::vector<float> fimg(img.begin(), img.end()), parts((size_t)n0);
        oracle_sample_image_max(&apr.d, &tree.d, 0, fimg.data(), nz, nx, ny, parts.data());
        check(parts, "sample_image_max");
        std::vector<uint16_t> labels(img.size());
        for (size_t i = 0; i < img.size(); ++i) labels[i] = img[i] > 400 ? (uint16_t)(1 + (i / 997) % 5) : 0;
        const float dzs[4] = {1.f, 0.f, 0.f, -0.5f}, dxs[4] = {0.f, 1.f, 0.f, 0.5f}, dys[4] = {0.f, 0.f, -1.f, 0.7f};
        std::vector<float> dist((size_t)n0 * 4);
        oracle_labels_to_dist_u16(&apr.d, &tree.d, 0, labels.data(), nz, nx, ny, dzs, dxs, dys, 4, 1 << 12, dist.data());
        check(dist, "labels_to_dist");
    }
    aprcore_destroy(h);
    std::printf("OK\n");
    return 0;
}
