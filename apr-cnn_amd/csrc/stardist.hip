// Label and coordinate utilities of the StarDist networks (pyapr/aprnet/src/utils.hpp:86-333), on the device:
// particle coordinates in pixels, sampling of a dense image onto the particles through a max pyramid, and the
// star-convex ray distances of a label image at every particle.  One launch per level, one workgroup per sparse
// row of that level; particles of levels <= Lc, then (level delta > 0) the downsampled particles of level Lc behind
// them, in the feature order of every other operator.
#include "common.hpp"

namespace aprnet {

// Centre of a particle's cell in pixels of the finest level: floor((c + 0.5) * 2^(level_max - level)),
// utils.hpp:108-110, 240-242.
__device__ __forceinline__ int cell_centre(int c, int shift) { return shift == 0 ? c : (c << shift) + (1 << (shift - 1)); }

// get_particle_coords (utils.hpp:222-267): coords[i] = (z, x, y) centre of particle i.
__global__ void __launch_bounds__(64)
coords_kernel(const AccessDev acc, int level, int shift, int64_t idx_off, float* __restrict__ coords) {
    const int x = blockIdx.x, z = blockIdx.y;
    const uint64_t row = acc.row(level, z, x);
    const int64_t b = (int64_t)acc.xz_end[row - 1], e = (int64_t)acc.xz_end[row];
    for (int64_t i = b + threadIdx.x; i < e; i += 64) {
        float* c = coords + (i + idx_off) * 3;
        c[0] = (float)cell_centre(z, shift);
        c[1] = (float)cell_centre(x, shift);
        c[2] = (float)cell_centre((int)acc.y[i], shift);
    }
}

// sample_image (utils.hpp:270-333): the value of a particle is the maximum of the image over its cell (the
// reference builds a pyramid by pairwise maxima; a cell's pyramid entry is the maximum over the pixels it covers,
// clipped at the far faces of the image).
__global__ void __launch_bounds__(64)
sample_max_kernel(const AccessDev acc, int level, int shift, int64_t idx_off, const float* __restrict__ img, int zn,
                  int xn, int yn, float* __restrict__ parts) {
    const int x = blockIdx.x, z = blockIdx.y;
    const int f = 1 << shift;
    const uint64_t row = acc.row(level, z, x);
    const int64_t b = (int64_t)acc.xz_end[row - 1], e = (int64_t)acc.xz_end[row];
    const int z0 = z * f, z1 = min(z0 + f, zn), x0 = x * f, x1 = min(x0 + f, xn);
    for (int64_t i = b + threadIdx.x; i < e; i += 64) {
        const int y0 = (int)acc.y[i] * f, y1 = min(y0 + f, yn);
        float m = -INFINITY;
        for (int zz = z0; zz < z1; ++zz)
            for (int xx = x0; xx < x1; ++xx)
                for (int yy = y0; yy < y1; ++yy) m = fmaxf(m, img[((int64_t)zz * xn + xx) * yn + yy]);
        parts[i + idx_off] = (z0 < z1 && x0 < x1 && y0 < y1) ? m : 0.f;
    }
}

// labels_to_dist_cpp (utils.hpp:86-219): for every particle whose centre lies in an object (label != 0) and every
// ray, step along the ray until the rounded position leaves the image or the object; the distance is the length of
// the rounded offset.  Same fp32 accumulation and round-half-even as the reference.  max_steps bounds the walk (a
// ray shorter than 1 / max_steps pixels per step would otherwise not end).
template <typename L>
__global__ void __launch_bounds__(64)
labels_to_dist_kernel(const AccessDev acc, int level, int shift, int64_t idx_off, const L* __restrict__ img, int zn, int xn,
                      int yn, const float* __restrict__ dzs, const float* __restrict__ dxs, const float* __restrict__ dys,
                      int n_rays, int max_steps, float* __restrict__ dist) {
    const int x = blockIdx.x, z = blockIdx.y;
    const uint64_t row = acc.row(level, z, x);
    const int64_t b = (int64_t)acc.xz_end[row - 1], e = (int64_t)acc.xz_end[row];
    const int ci = cell_centre(z, shift), cj = cell_centre(x, shift);
    if (ci >= zn || cj >= xn) return;
    const int64_t work = (e - b) * n_rays;
    for (int64_t w = threadIdx.x; w < work; w += 64) {
        const int64_t i = b + w / n_rays;
        const int n = (int)(w % n_rays);
        const int ck = cell_centre((int)acc.y[i], shift);
        if (ck >= yn) continue;
        const L value = img[((int64_t)ci * xn + cj) * yn + ck];
        if (value == 0) continue;
        const float dz = dzs[n], dx = dxs[n], dy = dys[n];
        float zz = 0.f, xx = 0.f, yy = 0.f;
        for (int step = 0; step < max_steps; ++step) {
            xx += dx; yy += dy; zz += dz;
            const int ii = __float2int_rn((float)ci + zz), jj = __float2int_rn((float)cj + xx), kk = __float2int_rn((float)ck + yy);
            if (ii < 0 || ii >= zn || jj < 0 || jj >= xn || kk < 0 || kk >= yn || img[((int64_t)ii * xn + jj) * yn + kk] != value)
                break;
        }
        zz = rintf(zz); xx = rintf(xx); yy = rintf(yy);
        dist[(i + idx_off) * n_rays + n] = sqrtf(xx * xx + yy * yy + zz * zz);
    }
}

// Launches `launch(access, level, shift, index offset)` for every level of the feature vector at `d`.
template <typename F>
static int for_each_level(const aprnet_plan* p, int d, const char* what, F launch) {
    if (int rc = check_level_delta(p, d, what)) return rc;
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    const int Lc = p->lc(d), lmax = p->apr.level_max;
    for (int l = Lc; l >= p->apr.level_min; --l) {
        if (p->apr.level_end(l) == p->apr.level_begin(l)) continue;
        launch(p->dapr, dim3((unsigned)p->apr.x_num[l], (unsigned)p->apr.z_num[l]), l, lmax - l, (int64_t)0);
    }
    if (d > 0 && p->tree.level_end(Lc) > p->tree.level_begin(Lc))
        launch(p->dtree, dim3((unsigned)p->tree.x_num[Lc], (unsigned)p->tree.z_num[Lc]), Lc, lmax - Lc, p->tree_offset(Lc));
    return 0;
}

static int check_image(const aprnet_plan* p, int zn, int xn, int yn, const char* what) {
    const int l = p->apr.level_max;
    if (zn != p->apr.z_num[l] || xn != p->apr.x_num[l] || yn != p->apr.y_num[l])
        return fail(APRNET_ERR_INVALID_ARGUMENT, std::string(what) + ": the image must have the shape of the APR's finest level");
    return 0;
}

template <typename L>
static int labels_to_dist(const aprnet_plan* p, int d, const L* img, int zn, int xn, int yn, const float* dzs, const float* dxs,
                          const float* dys, int n_rays, int max_steps, float* dist, hipStream_t st) {
    if (!p || !img || !dzs || !dxs || !dys || !dist || n_rays <= 0 || max_steps <= 0)
        return fail(APRNET_ERR_INVALID_ARGUMENT, "labels_to_dist: null argument or no rays");
    if (int rc = check_image(p, zn, xn, yn, "labels_to_dist")) return rc;
    int rc = for_each_level(p, d, "labels_to_dist", [&](const AccessDev& acc, dim3 grid, int l, int shift, int64_t off) {
        hipLaunchKernelGGL(labels_to_dist_kernel<L>, grid, dim3(64), 0, st, acc, l, shift, off, img, zn, xn, yn, dzs, dxs, dys,
                           n_rays, max_steps, dist);
    });
    if (rc) return rc;
    APRNET_LAUNCH_CHECK("labels_to_dist_kernel");
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
int aprnet_particle_coords(const aprnet_plan* p, int d, float* coords, void* st) {
    if (!p || !coords) return fail(APRNET_ERR_INVALID_ARGUMENT, "particle_coords: null argument");
    int rc = for_each_level(p, d, "particle_coords", [&](const AccessDev& acc, dim3 grid, int l, int shift, int64_t off) {
        hipLaunchKernelGGL(coords_kernel, grid, dim3(64), 0, (hipStream_t)st, acc, l, shift, off, coords);
    });
    if (rc) return rc;
    APRNET_LAUNCH_CHECK("coords_kernel");
    return 0;
}
int aprnet_sample_image_max_f32(const aprnet_plan* p, int d, const float* img, int zn, int xn, int yn, float* parts, void* st) {
    if (!p || !img || !parts) return fail(APRNET_ERR_INVALID_ARGUMENT, "sample_image: null argument");
    if (int rc = check_image(p, zn, xn, yn, "sample_image")) return rc;
    int rc = for_each_level(p, d, "sample_image", [&](const AccessDev& acc, dim3 grid, int l, int shift, int64_t off) {
        hipLaunchKernelGGL(sample_max_kernel, grid, dim3(64), 0, (hipStream_t)st, acc, l, shift, off, img, zn, xn, yn, parts);
    });
    if (rc) return rc;
    APRNET_LAUNCH_CHECK("sample_max_kernel");
    return 0;
}
#define LABELS_API(T, SFX)                                                                                               \
    int aprnet_labels_to_dist_##SFX(const aprnet_plan* p, int d, const T* img, int zn, int xn, int yn, const float* dzs,  \
                                    const float* dxs, const float* dys, int n_rays, int max_steps, float* dist, void* st) { \
        return labels_to_dist<T>(p, d, img, zn, xn, yn, dzs, dxs, dys, n_rays, max_steps, dist, (hipStream_t)st); }
LABELS_API(uint8_t, u8)
LABELS_API(uint16_t, u16)
LABELS_API(uint32_t, u32)
LABELS_API(uint64_t, u64)
}
