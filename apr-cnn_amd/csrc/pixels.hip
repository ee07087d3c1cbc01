// Particles <-> dense image at the resolution of the current maximum level Lc:
// reconstruct_forward/backward (cuda/src/reconstruct_gpu.cu:3-127) and sample_particles_forward/backward
// (cuda/src/sample_particles_gpu.cu:3-145).  One launch per level, one workgroup per sparse row of that
// level, one thread per particle, which walks its own f x f x f cell (f = 2^(Lc-level), clipped at the
// image border).  A particle is the only writer of its cell and the only reader of its sums, so none
// of the four directions needs atomics (the reference accumulates with atomicAdd across row blocks).
#include "common.hpp"

namespace aprnet {

enum PixelMode { RECON_FWD = 0, RECON_BWD = 1, SAMPLE_FWD = 2, SAMPLE_BWD = 3 };

template <typename T, int MODE>
__global__ void __launch_bounds__(64)
pixel_kernel(const AccessDev acc, int level, int Lc, int64_t idx_off, T* __restrict__ parts, int64_t ldp, int C,
             T* __restrict__ img, int64_t ldi) {
    const int x = blockIdx.x, z = blockIdx.y;
    const int f = 1 << (Lc - level);
    const int zn = acc.z_num[Lc], xn = acc.x_num[Lc], yn = acc.y_num[Lc];
    const uint64_t row = acc.row(level, z, x);
    const int64_t b = (int64_t)acc.xz_end[row - 1], e = (int64_t)acc.xz_end[row];
    const int z0 = z * f, z1 = min(z0 + f, zn), x0 = x * f, x1 = min(x0 + f, xn);
    for (int64_t i = b + threadIdx.x; i < e; i += 64) {
        const int y0 = (int)acc.y[i] * f, y1 = min(y0 + f, yn);
        typedef typename Num<T>::acc A;     // bfloat16 cells are summed and divided in fp32
        for (int c = 0; c < C; ++c) {
            T* pv = parts + (int64_t)c * ldp + i + idx_off;
            T* im = img + (int64_t)c * ldi;
            if (MODE == RECON_FWD || MODE == SAMPLE_BWD) {
                const T v = MODE == RECON_FWD ? *pv : Num<T>::st(Num<T>::ld(*pv) / (A)((z1 - z0) * (x1 - x0) * (y1 - y0)));
                for (int zz = z0; zz < z1; ++zz)
                    for (int xx = x0; xx < x1; ++xx)
                        for (int yy = y0; yy < y1; ++yy) im[((int64_t)zz * xn + xx) * yn + yy] = v;
            } else {
                A s = 0;
                for (int zz = z0; zz < z1; ++zz)
                    for (int xx = x0; xx < x1; ++xx)
                        for (int yy = y0; yy < y1; ++yy) s += Num<T>::ld(im[((int64_t)zz * xn + xx) * yn + yy]);
                *pv = Num<T>::st(MODE == RECON_BWD ? s : s / (A)((z1 - z0) * (x1 - x0) * (y1 - y0)));
            }
        }
    }
}

template <typename T, int MODE>
int pixel_op(const aprnet_plan* p, int d, T* parts, int64_t ldp, int C, T* img, int64_t ldi, hipStream_t st) {
    if (int rc = check_level_delta(p, d, "reconstruct/sample")) return rc;
    if (C <= 0) return 0;
    if (int rc = check_rows(ldp, p->number_parts(d), "reconstruct/sample", "particle tensor")) return rc;
    APRNET_HIP_CHECK(hipSetDevice(p->device));
    const int Lc = p->lc(d);
    if (int rc = check_rows(ldi, (int64_t)p->apr.z_num[Lc] * p->apr.x_num[Lc] * p->apr.y_num[Lc], "reconstruct/sample", "image")) return rc;
    for (int l = Lc; l >= p->apr.level_min; --l) {
        if (p->apr.level_end(l) == p->apr.level_begin(l)) continue;
        dim3 grid((unsigned)p->apr.x_num[l], (unsigned)p->apr.z_num[l]);
        hipLaunchKernelGGL((pixel_kernel<T, MODE>), grid, dim3(64), 0, st, p->dapr, l, Lc, (int64_t)0, parts, ldp, C, img, ldi);
    }
    if (d > 0 && p->tree.level_end(Lc) > p->tree.level_begin(Lc)) {     // downsampled particles
        dim3 grid((unsigned)p->tree.x_num[Lc], (unsigned)p->tree.z_num[Lc]);
        hipLaunchKernelGGL((pixel_kernel<T, MODE>), grid, dim3(64), 0, st, p->dtree, Lc, Lc, p->tree_offset(Lc), parts, ldp, C, img, ldi);
    }
    APRNET_LAUNCH_CHECK("pixel_kernel");
    return 0;
}

}  // namespace aprnet

using namespace aprnet;
extern "C" {
#define PIXEL_API(T, SFX)                                                                                              \
    int aprnet_reconstruct_fwd_##SFX(const aprnet_plan* p, int d, const T* x, int64_t ldx, int C, T* img, int64_t ldi, \
                                     void* st) { return pixel_op<T, RECON_FWD>(p, d, const_cast<T*>(x), ldx, C, img, ldi, (hipStream_t)st); } \
    int aprnet_reconstruct_bwd_##SFX(const aprnet_plan* p, int d, const T* gimg, int64_t ldi, int C, T* gx, int64_t ldx, \
                                     void* st) { return pixel_op<T, RECON_BWD>(p, d, gx, ldx, C, const_cast<T*>(gimg), ldi, (hipStream_t)st); } \
    int aprnet_sample_particles_fwd_##SFX(const aprnet_plan* p, int d, const T* img, int64_t ldi, int C, T* y, int64_t ldy, \
                                          void* st) { return pixel_op<T, SAMPLE_FWD>(p, d, y, ldy, C, const_cast<T*>(img), ldi, (hipStream_t)st); } \
    int aprnet_sample_particles_bwd_##SFX(const aprnet_plan* p, int d, const T* gy, int64_t ldy, int C, T* gimg, int64_t ldi, \
                                          void* st) { return pixel_op<T, SAMPLE_BWD>(p, d, const_cast<T*>(gy), ldy, C, gimg, ldi, (hipStream_t)st); }
PIXEL_API(float, f32)
PIXEL_API(double, f64)
// bfloat16 images and particles (bit patterns in uint16_t): sums and means in fp32, rounded to nearest even on store
int aprnet_reconstruct_fwd_bf16(const aprnet_plan* p, int d, const uint16_t* x, int64_t ldx, int C, uint16_t* img, int64_t ldi, void* st) {
    return pixel_op<bf16_t, RECON_FWD>(p, d, (bf16_t*)const_cast<uint16_t*>(x), ldx, C, (bf16_t*)img, ldi, (hipStream_t)st); }
int aprnet_reconstruct_bwd_bf16(const aprnet_plan* p, int d, const uint16_t* gimg, int64_t ldi, int C, uint16_t* gx, int64_t ldx, void* st) {
    return pixel_op<bf16_t, RECON_BWD>(p, d, (bf16_t*)gx, ldx, C, (bf16_t*)const_cast<uint16_t*>(gimg), ldi, (hipStream_t)st); }
int aprnet_sample_particles_fwd_bf16(const aprnet_plan* p, int d, const uint16_t* img, int64_t ldi, int C, uint16_t* y, int64_t ldy, void* st) {
    return pixel_op<bf16_t, SAMPLE_FWD>(p, d, (bf16_t*)y, ldy, C, (bf16_t*)const_cast<uint16_t*>(img), ldi, (hipStream_t)st); }
int aprnet_sample_particles_bwd_bf16(const aprnet_plan* p, int d, const uint16_t* gy, int64_t ldy, int C, uint16_t* gimg, int64_t ldi, void* st) {
    return pixel_op<bf16_t, SAMPLE_BWD>(p, d, (bf16_t*)const_cast<uint16_t*>(gy), ldy, C, (bf16_t*)gimg, ldi, (hipStream_t)st); }
}
