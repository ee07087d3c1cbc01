/* aprnet_hip.h — C ABI of the MI355X (gfx950) particle-space CNN operators.
 *
 * Drop-in boundary for the native functions that APR-CNN registers on
 * `_pyaprwrapper.aprnet.{conv,pool,upsample,utils,cuda}` (wrappers/pythonBind.cpp:144-182).
 * Each entry point below names the reference function it replaces.
 *
 * Conventions
 *  - Every function returns 0 on success and a negative aprnet_status otherwise; the message of
 *    the last failure on the calling thread is available from aprnet_last_error().  Nothing throws.
 *  - An `aprnet_plan` is the device-side image of one APR (what `APR::init_cuda()` /
 *    `GPUAccessHelper` is in the reference, wrap_conv_gpu.hpp:23-28): the access arrays plus the
 *    child table and tile lists derived from them.  It is created from HOST arrays and owns its
 *    device memory.  All other pointers are DEVICE pointers owned by the caller.
 *  - Operators work on ONE batch item: features are `C` channel planes of `n` particles, plane `c`
 *    starting at `base + c*ld` (ld in elements).  The reference's batch loop
 *    (conv.hpp:99, wrap_conv_gpu.hpp:23-28) stays on the caller's side.  Every `ld` is checked against the
 *    number of elements the operator touches per channel at its level delta (aprnet_number_parts, the tree
 *    size, the image size) before anything is launched: a shorter row is APRNET_ERR_INVALID_ARGUMENT with
 *    both numbers in the message, as the reference refuses tensors whose shape does not match (conv.hpp:63-66).
 *  - Work-space contents: the stencil convolutions fill the mean tree in `tree_ws` only at the nodes their
 *    kernels read (the others keep what the buffer held); callers must not rely on it afterwards.
 *  - `level_delta` d is the number of finest levels pooled away (helpers.hpp:86-117);
 *    Lc = level_max - d.  A feature vector at d holds aprnet_number_parts(plan, d) values.
 *  - No function allocates caller-visible memory; work space is passed in.  Kernels are enqueued
 *    on `stream` (a hipStream_t passed as void*) and the call returns without synchronising.
 *  - Suffix _f32 / _f64 = element type of features, weights and gradients.
 */
#ifndef APRNET_HIP_H
#define APRNET_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum aprnet_status {
    APRNET_OK = 0,
    APRNET_ERR_INVALID_ARGUMENT = -1,   /* std::invalid_argument in the reference (conv.hpp:63-66, upsample.hpp:49-54) */
    APRNET_ERR_LEVEL_DELTA = -2,        /* CHECK_LEVEL_DELTA (cuda/src/common.hpp:17) */
    APRNET_ERR_HIP = -3,                /* a HIP runtime call failed */
    APRNET_ERR_UNSUPPORTED = -4
} aprnet_status;

/* One linear access structure, as LibAPR's LinearAccess / GPUAccessHelper expose it
 * (row lookup idiom: conv333_gpu.cu:65-67; state: data_containers/src/BindAPR.hpp:72-108).
 * All pointers are host pointers; the arrays are copied. */
typedef struct aprnet_access_desc {
    int32_t level_min, level_max;
    const int32_t* z_num;            /* indexed by level; [L+1] entries with L = level_max of the APR's own access */
                                     /* (also in the tree's descriptor, whose level_max is L-1)                */
    const int32_t* x_num;
    const int32_t* y_num;
    const uint64_t* level_xz_vec;    /* [level_max+2] */
    const uint64_t* xz_end_vec;      /* [n_rows] with leading sentinel 0 */
    const uint16_t* y_vec;           /* [n_particles]; per row strictly ascending and < y_num of the row's level */
    uint64_t n_rows;
    uint64_t n_particles;
} aprnet_access_desc;

typedef struct aprnet_plan aprnet_plan;

const char* aprnet_last_error(void);

/* Replaces APR::init_cuda() + gpuAPRHelper()/gpuTreeHelper() (wrap_conv_gpu.hpp:25-26).  The arrays are validated on
 * the host (row table non-decreasing and within n_particles, level_xz_vec consistent with z_num * x_num, y strictly
 * ascending per row and below y_num): APRNET_ERR_INVALID_ARGUMENT names the first violation. */
int aprnet_plan_create(const aprnet_access_desc* apr, const aprnet_access_desc* tree, int device, aprnet_plan** out);
void aprnet_plan_destroy(aprnet_plan* plan);

/* No counterpart in the reference.  The convolutions keep re-laid-out weights (and, for bfloat16 features, a regrouped
 * copy of their input) in one scratch buffer of the plan that grows to the largest call seen.  Growth allocates, so it is
 * refused with APRNET_ERR_UNSUPPORTED while `stream` is capturing into a graph, and so is the first convolution at a
 * level delta (it builds the plan's tile and window lists).  Call this - or run the network once - before a capture;
 * a buffer that a captured graph may address is kept until aprnet_plan_destroy.  Calls that share a plan use one
 * stream at a time: a call on another stream first waits for the previous one. */
int aprnet_plan_reserve(aprnet_plan* plan, int64_t bytes, void* stream);

/* helpers::number_parts (helpers.hpp:86-101); also number_parts_after_pooling/_upsampling with d±1. */
int64_t aprnet_number_parts(const aprnet_plan* plan, int level_delta);
/* helpers::compute_tree_offset (helpers.hpp:113-117) for `level`. */
int64_t aprnet_tree_offset(const aprnet_plan* plan, int level);
/* tree_it.total_number_particles(Lc-1): length of the tree work space at d (helpers.hpp:166). */
int64_t aprnet_tree_parts(const aprnet_plan* plan, int level_delta);
/* Copies the child table to host: int32 [8][n_tree]; slot s = 4*dz+2*dx+dy of tree node t holds the
 * particle index (>= 0), ~tree_index (< 0, != INT32_MIN) or INT32_MIN when the child cell lies outside
 * the image.  This is the index map behind the parent walks of helpers.hpp:185-194, maxpool.hpp:106-117,
 * upsample.hpp:112-118. */
int aprnet_plan_children(const aprnet_plan* plan, int32_t* out_host);

/* No counterpart in the reference (it has no profiling hooks).
 * When enabled, the main kernel of every aprnet_conv_fwd_* call is bracketed by two HIP events recorded on
 * the call's stream; aprnet_profile_last_ms() waits for the last bracket and returns its duration in
 * milliseconds (-1 if none).  Process-wide, not thread-safe; meant for benchmarks. */
int aprnet_profile_enable(int on);
/* No counterpart in the reference.  A knob for TESTS AND MEASUREMENTS, not part of the operator interface: it selects
 * between kernels that compute the same results, process-wide (atomic flags; a call in flight keeps the choice it read),
 * so that tests can cover every kernel family and benchmarks can compare them.  Callers of the operators never need it,
 * and it answers only in a process started with APRNET_TESTING=1 in its environment (read once, at the first call);
 * everywhere else it returns APRNET_ERR_UNSUPPORTED and changes nothing.
 * Selects the convolution kernels: 0 = matrix-core (MFMA) kernels where one
 * exists for the stencil and element type, VALU kernels otherwise (default); 1 = VALU kernels only.
 * Independently, for bfloat16 features: 2 = bfloat16 matrix instructions (default), 3 = fp32 matrix
 * instructions; and for the forward matrix-core kernels: 4 = take the window lists that the plan builds on first
 * use and keeps (about 20 bytes of device memory per particle and level delta; default), 5 = scan the access arrays
 * in every call (also the fallback when the lists cannot be allocated); and for the backward matrix-core kernels:
 * 6 = the weight gradient runs on a second stream of the plan next to the input gradient, forked from and joined
 * to the caller's stream with events (default), 7 = both on the caller's stream; and for the bfloat16 forward
 * kernel: 8 = stage from a copy of the input regrouped as [Cin / 8][particles][8] in the plan's scratch buffer, one
 * 16-byte load per item and 8 channels (default; 16 bytes per particle and 8 channels of device memory, made by one
 * streaming pass per call), 9 = gather from the channel planes; and for the weight gradient of the matrix-core
 * kernels: 10 = every workgroup writes the sums of its tiles to its own slots of the plan's scratch buffer and a second
 * kernel adds the slots in a fixed order (default: the gradient repeats bit for bit from run to run; at most 512 MiB
 * of scratch), 11 = atomic additions; and for forward layers of 1 to 3 input channels (bound by memory, not by the
 * contraction): 12 = the pipelined kernel with the (tap, channel) axis flattened (default), 13 = the general kernel;
 * and for the bfloat16 forward kernel on grouped tensors: 14 = 32-bit byte offsets where a group holds fewer than 2^28
 * elements, 64-bit addresses beyond (default), 15 = 64-bit addresses always; and for the tree fill that precedes a
 * forward stencil convolution: 16 = fill the nodes that the kernel's window lists read, and their descendants (default;
 * the node lists are built with the window lists and kept in the plan, 4 bytes per needed node), 17 = fill every node.
 * All are HIP kernels; the switch
 * exists so that tests can cover them and memory-bound callers can do without the lists. */
int aprnet_set_conv_path(int path);
float aprnet_profile_last_ms(void);

/* Bias gradient of a convolution: out[c] (+)= sum_i x[c*ld + i], i < n (replaces torch.sum(grad_output, dim=(0, 2)),
 * conv.py:33, cuda/conv.py:33, one batch item per call; pass accumulate != 0 for the items after the first).
 * Two passes in a fixed order, no atomics.  work: aprnet_channel_sum_work_elems(C) elements of scratch. */
int aprnet_channel_sum_work_elems(int C);
int aprnet_channel_sum_f32(const float* x, int64_t ld, int C, int64_t n, float* out, int accumulate, float* work, void* stream);
int aprnet_channel_sum_f64(const double* x, int64_t ld, int C, int64_t n, double* out, int accumulate, double* work, void* stream);

/* No counterpart in the reference: aprnet_channel_sum_f32 for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The block partials that the other entry point
 * keeps in the caller's `work` live in a 1 MiB device array of this library (one copy per GPU, held until the
 * process ends); the call allocates nothing and frees nothing.  The current device must be the one x and out live on.
 * At most aprnet_channel_sum_static_max_channels() (1024) channels per call: APRNET_ERR_UNSUPPORTED beyond.  All calls
 * on one GPU share the array: calls that overlap on one GPU (two streams) race and must be ordered by the caller. */
int aprnet_channel_sum_static_max_channels(void);
int aprnet_channel_sum_static_f32(const float* x, int64_t ld, int C, int64_t n, float* out, int accumulate, void* stream);

/* Optional parts of aprnet_conv_fwd_fused_*.  They fuse what the reference network does in separate passes around
 * a convolution: torch.cat of the skip connection and the upsampled features before the first convolution of a
 * decoder stage (unet_parts.py:82), and the ReLU that follows a convolution whose norm has been folded into it
 * (BasicBlock, unet_parts.py:17-26). */
typedef struct aprnet_conv_fusion {
    const void* x2;   /* second input [C2][ldx2], element type of x: its channels follow the Cin channels of x in   */
    int64_t ldx2;     /* the contraction, i.e. w has Cin + C2 input channels; NULL / 0 for a single input           */
    int32_t C2;
    int32_t relu;     /* nonzero: y = max(conv + bias, 0) */
    const void* x2_coarse; /* grouped bfloat16 inputs only (aprnet_conv_fwd_fused_bf16l, aprnet_conv_fwd_head_bf16g), else NULL:  */
    int64_t ld_coarse;     /* the tensor [C2 / 8][ld_coarse][8] at level_delta + 1 that x2 is the UpSampleConst of              */
                           /* (UpConv.forward, unet_parts.py:79-83).  The mean tree of an upsampled tensor holds the values it   */
                           /* was upsampled from, so the tree of x2 is taken from x2_coarse (an eighth of the values to read)   */
                           /* instead of computed from x2; same results.  x2 itself is still read for the particles.             */
} aprnet_conv_fusion;

#define APRNET_DECL(T, SFX)                                                                                          \
    /* helpers::fill_tree_mean (helpers.hpp:156-252): tree[c][t] for all tree nodes of level < Lc. */               \
    int aprnet_fill_tree_mean_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int C,            \
                                    T* tree, int64_t ld_tree, void* stream);                                        \
    /* helpers::fill_tree_mean_backward (helpers.hpp:255-350): pushes grad_tree root->leaf (grad_tree is            \
     * modified) and ACCUMULATES into grad_x. */                                                                    \
    int aprnet_fill_tree_mean_bwd_##SFX(const aprnet_plan*, int level_delta, T* grad_x, int64_t ldx, int C,         \
                                        T* grad_tree, int64_t ld_tree, void* stream);                               \
    /* Convolution<kz,kx,ky>::forward (conv.hpp:55-195), CUDA twin conv333_forward (wrap_conv_gpu.hpp:32-66).       \
     * (kz,kx,ky) in {333,133,155,555}.  w: expanded stencils [S_exp][Cout][Cin][kz][kx][ky] (the layout of         \
     * cuda/conv.py:77).  y is OVERWRITTEN for indices < number_parts(d).  bias: [Cout] or NULL; the reference     \
     * adds it in a separate pass (conv.py:101), here it is fused into the store.  tree_ws: [Cin][ld_tree]         \
     * scratch, ld_tree >= aprnet_tree_parts(plan, d). */                                                           \
    int aprnet_conv_fwd_##SFX(const aprnet_plan*, int level_delta, int kz, int kx, int ky,                          \
                              const T* x, int64_t ldx, int Cin, const T* w, int S_exp, int Cout, const T* bias,     \
                              T* y, int64_t ldy, T* tree_ws, int64_t ld_tree, void* stream);                        \
    /* The same with the optional fused parts (fusion may be NULL).  With a second input tree_ws is                 \
     * [Cin + C2][ld_tree].  (kz,kx,ky) = (1,1,1) is accepted too (w [S][Cout][Cin], no second input, tree_ws       \
     * unused): Convolution<1,1,1>::forward followed by the ReLU. */                                                \
    int aprnet_conv_fwd_fused_##SFX(const aprnet_plan*, int level_delta, int kz, int kx, int ky,                    \
                                    const T* x, int64_t ldx, int Cin, const T* w, int S_exp, int Cout,              \
                                    const T* bias, T* y, int64_t ldy, T* tree_ws, int64_t ld_tree,                  \
                                    const aprnet_conv_fusion* fusion, void* stream);                                \
    /* Convolution<kz,kx,ky>::backward (conv.hpp:261-481), CUDA twin conv333_backward.  grad_x is OVERWRITTEN,      \
     * grad_w [S_exp][Cout][Cin][k] is ACCUMULATED into (zero it before the first batch item, as                    \
     * torch::zeros_like does in conv.hpp:270).  tree_ws / grad_tree_ws: [Cin][ld_tree] scratch each.               \
     * grad_x may be NULL (no counterpart in the reference: the first layer of a network needs no input gradient):  \
     * then only grad_w is computed and grad_tree_ws is not used. */                                                \
    int aprnet_conv_bwd_##SFX(const aprnet_plan*, int level_delta, int kz, int kx, int ky,                          \
                              const T* x, int64_t ldx, int Cin, const T* w, int S_exp, int Cout,                    \
                              const T* grad_y, int64_t ldy, T* grad_x, int64_t ldgx, T* grad_w,                     \
                              T* tree_ws, int64_t ld_tree, T* grad_tree_ws, int64_t ld_gtree, void* stream);        \
    /* Convolution<1,1,1>::forward/backward (conv.hpp:199-256, 484-554); w: [S][Cout][Cin] (not expanded,           \
     * stencil index min(S-1, Lc-level)).  grad_w is accumulated, grad_x overwritten. */                            \
    int aprnet_conv111_fwd_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int Cin,             \
                                 const T* w, int S, int Cout, const T* bias, T* y, int64_t ldy, void* stream);      \
    int aprnet_conv111_bwd_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int Cin,             \
                                 const T* w, int S, int Cout, const T* grad_y, int64_t ldy,                         \
                                 T* grad_x, int64_t ldgx, T* grad_w, void* stream);                                 \
    /* MaxPool::forward (maxpool.hpp:43-146): y[c][0:number_parts(d+1)], argmax = INPUT index, ties resolved in     \
     * the CPU traversal order (z, x, y; particles before downsampled particles; strict >). */                     \
    int aprnet_maxpool_fwd_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int C,               \
                                 T* y, int64_t ldy, int64_t* argmax, int64_t ldi, void* stream);                    \
    /* MaxPool::backward (maxpool.hpp:149-230): grad_x[0:number_parts(d)] overwritten. */                          \
    int aprnet_maxpool_bwd_##SFX(const aprnet_plan*, int level_delta, const T* grad_y, int64_t ldy, int C,          \
                                 T* grad_x, int64_t ldx, const int64_t* argmax, int64_t ldi, void* stream);         \
    /* UpSampleConst::forward/backward (upsample.hpp:39-236); level_delta is that of the INPUT (> 0). */           \
    int aprnet_upsample_fwd_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int C,              \
                                  T* y, int64_t ldy, void* stream);                                                 \
    int aprnet_upsample_bwd_##SFX(const aprnet_plan*, int level_delta, const T* grad_y, int64_t ldy, int C,         \
                                  T* grad_x, int64_t ldx, void* stream);                                            \
    /* RestrictKernel<kz,kx,ky>::forward/backward (kernel.hpp:31-224) on [S][Cout][Cin][k] weights:                 \
     * w [S][n_filters][k] -> w_exp [S_exp][n_filters][k] with n_filters = Cout*Cin; backward is the transpose. */  \
    int aprnet_restrict_kernel_fwd_##SFX(const T* w, int S, int n_filters, int kz, int kx, int ky, int S_exp,       \
                                         T* w_exp, void* stream);                                                   \
    int aprnet_restrict_kernel_bwd_##SFX(const T* grad_w_exp, int S_exp, int n_filters, int kz, int kx, int ky,     \
                                         int S, T* grad_w, void* stream);                                           \
    /* reconstruct_forward/backward (cuda/src/reconstruct_gpu.cu:3-197): particles -> dense                         \
     * [C][z_num(Lc)][x_num(Lc)][y_num(Lc)], plane stride ld_img; cells no particle covers keep their value. */     \
    int aprnet_reconstruct_fwd_##SFX(const aprnet_plan*, int level_delta, const T* x, int64_t ldx, int C,           \
                                     T* img, int64_t ld_img, void* stream);                                         \
    int aprnet_reconstruct_bwd_##SFX(const aprnet_plan*, int level_delta, const T* grad_img, int64_t ld_img, int C, \
                                     T* grad_x, int64_t ldx, void* stream);                                         \
    /* sample_particles_forward/backward (cuda/src/sample_particles_gpu.cu:3-246): dense -> particles (cell mean). */\
    int aprnet_sample_particles_fwd_##SFX(const aprnet_plan*, int level_delta, const T* img, int64_t ld_img, int C, \
                                          T* y, int64_t ldy, void* stream);                                         \
    int aprnet_sample_particles_bwd_##SFX(const aprnet_plan*, int level_delta, const T* grad_y, int64_t ldy, int C, \
                                          T* grad_img, int64_t ld_img, void* stream);

APRNET_DECL(float, f32)
APRNET_DECL(double, f64)

/* bfloat16 features (uint16_t bit patterns; no counterpart in the reference, which has no 16-bit path).
 * Values are widened to fp32 on load, accumulated in fp32 and rounded to nearest even on store.  Weights
 * and bias are passed in fp32; the stencil convolution (3x3x3, 1x3x3, 1x5x5) rounds the weights to bfloat16
 * and multiplies on the bfloat16 matrix cores (aprnet_set_conv_path(3) keeps the weights and the products
 * in fp32; layers of 2 or 3 input channels, and one-channel layers of the 2-D stencils, keep fp32 weights and
 * products; the 5x5x5 stencil has no matrix-core kernel and multiplies in fp32 on the vector-ALU kernel, forward
 * only).  Forward operators of the APR-UNet, plus the backward passes
 * of pool / upsample / tree fill and of the stencil convolution.  Argument meaning as
 * for the _f32 entry points. */
int aprnet_conv_fwd_bf16(const aprnet_plan*, int level_delta, int kz, int kx, int ky, const uint16_t* x, int64_t ldx, int Cin,
                         const float* w, int S_exp, int Cout, const float* bias, uint16_t* y, int64_t ldy,
                         uint16_t* tree_ws, int64_t ld_tree, void* stream);          /* 5x5x5: fp32 products on the vector-ALU kernel */
int aprnet_conv_fwd_fused_bf16(const aprnet_plan*, int level_delta, int kz, int kx, int ky, const uint16_t* x, int64_t ldx,
                               int Cin, const float* w, int S_exp, int Cout, const float* bias, uint16_t* y, int64_t ldy,
                               uint16_t* tree_ws, int64_t ld_tree, const aprnet_conv_fusion* fusion, void* stream);
int aprnet_conv111_fwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int Cin, const float* w,
                            int S, int Cout, const float* bias, uint16_t* y, int64_t ldy, void* stream);
/* Convolution<1,1,1>::backward with bfloat16 features and output gradient: fp32 weights, fp32 weight gradient
 * (accumulated into gw), fp32 accumulation; gx overwritten.  At most 128 output channels. */
int aprnet_conv111_bwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int Cin, const float* w,
                            int S, int Cout, const uint16_t* gy, int64_t ldy, uint16_t* gx, int64_t ldgx, float* gw,
                            void* stream);
int aprnet_fill_tree_mean_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* tree,
                               int64_t ld_tree, void* stream);
int aprnet_fill_tree_mean_bwd_bf16(const aprnet_plan*, int level_delta, uint16_t* gx, int64_t ldx, int C, uint16_t* gtree,
                                   int64_t ld_tree, void* stream);
int aprnet_maxpool_fwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy,
                            int64_t* argmax, int64_t ldi, void* stream);
int aprnet_maxpool_bwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* gy, int64_t ldy, int C, uint16_t* gx,
                            int64_t ldx, const int64_t* argmax, int64_t ldi, void* stream);
int aprnet_upsample_fwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* y,
                             int64_t ldy, void* stream);
/* reconstruct / sample_particles with bfloat16 particles and images (cuda/src/reconstruct_gpu.cu:3-127,
 * sample_particles_gpu.cu:3-246; the reference has no 16-bit path): cell sums and means in fp32. */
int aprnet_reconstruct_fwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* img,
                                int64_t ld_img, void* stream);
int aprnet_reconstruct_bwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* grad_img, int64_t ld_img, int C, uint16_t* grad_x,
                                int64_t ldx, void* stream);
int aprnet_sample_particles_fwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* img, int64_t ld_img, int C, uint16_t* y,
                                     int64_t ldy, void* stream);
int aprnet_sample_particles_bwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* grad_y, int64_t ldy, int C, uint16_t* grad_img,
                                     int64_t ld_img, void* stream);
/* Backward of the stencil convolution with bfloat16 features and output gradient: fp32 weights, fp32 weight
 * gradient (accumulated into gw), fp32 accumulation everywhere; the input gradient is collected in the fp32 work
 * space gx32_ws [Cin][ld_gx32] (ld_gx32 >= aprnet_number_parts) and rounded to bfloat16 into gx at the end.
 * gtree_ws: fp32 [Cin][ld_gtree].  The input gradient multiplies on the bfloat16 matrix cores (weights rounded to
 * bfloat16) from input-gradient lists that the plan builds on first use; with aprnet_set_conv_path(3) or (5) it
 * runs with fp32 products and scans per call.  The weight gradient multiplies on the bfloat16 matrix cores as well
 * (both operands are bfloat16 as stored, so the products are exact), or with fp32 instructions under path 3.  gx may be NULL:
 * then only gw is computed and gx32_ws / gtree_ws are not used. */
int aprnet_conv_bwd_bf16(const aprnet_plan*, int level_delta, int kz, int kx, int ky, const uint16_t* x, int64_t ldx, int Cin,
                         const float* w, int S_exp, int Cout, const uint16_t* gy, int64_t ldy, uint16_t* gx, int64_t ldgx,
                         float* gw, uint16_t* tree_ws, int64_t ld_tree, float* gx32_ws, int64_t ld_gx32, float* gtree_ws,
                         int64_t ld_gtree, void* stream);
int aprnet_channel_sum_bf16(const uint16_t* x, int64_t ld, int C, int64_t n, float* out, int accumulate, float* work, void* stream);
int aprnet_upsample_bwd_bf16(const aprnet_plan*, int level_delta, const uint16_t* gy, int64_t ldy, int C, uint16_t* gx,
                             int64_t ldx, void* stream);

/* bfloat16 features grouped by eight channels: [C / 8][ld][8], the eight channels of a particle in one 16-byte word
 * (no counterpart in the reference, whose tensors are channel planes, conv.hpp:68).  A network's forward pass that
 * hands grouped tensors from layer to layer converts at its two ends only; the convolution then stages straight from
 * its input (no regrouping pass per call) and stores 8 bytes per lane instead of four 2-byte values.  Results are
 * bit-identical to the plane entry points (same arithmetic, same summation order).  C, Cin and Cout of grouped
 * tensors are multiples of 8; ld counts particles between two groups; at most 2^31 - 1 particles (from 2^28 on the
 * convolution addresses its 16-byte items with 64 bits instead of 32-bit byte offsets).
 *   regroup8 / ungroup8     planes [C][ldx] <-> groups [C / 8][ldo][8] (channels past C read as zeros)
 *   fill_tree_mean_bf16g    helpers::fill_tree_mean on grouped features, tree [C / 8][ld_tree][8]
 *   maxpool_fwd_bf16g       MaxPool::forward, values only (the argmax serves the backward pass)
 *   upsample_fwd_bf16g      UpSampleConst::forward
 *   conv111_fwd_bf16g       Convolution<1,1,1>::forward with bias and optional ReLU; y grouped (y_grouped != 0) or planes
 *                           (the head of a network); at most 256 inputs.  Layers of 16 to 128
 *                           inputs, multiply on the bfloat16 matrix cores with each fp32 weight split into a bfloat16
 *                           head and remainder (weights kept to 2^-16, sums in fp32); smaller layers multiply in fp32
 *   conv_fwd_fused_bf16l    aprnet_conv_fwd_fused_bf16 with a layout per tensor: x (and fusion->x2) grouped, or planes
 *                           of 1 to 3 channels; y grouped or planes; tree_ws has the layout of x */
int aprnet_regroup8_bf16(const uint16_t* x, int64_t ldx, int C, int64_t n, uint16_t* out, int64_t ldo, void* stream);
int aprnet_ungroup8_bf16(const uint16_t* xg, int64_t ldg, int C, int64_t n, uint16_t* out, int64_t ldo, void* stream);
int aprnet_fill_tree_mean_bf16g(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* tree,
                                int64_t ld_tree, void* stream);
int aprnet_maxpool_fwd_bf16g(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy,
                             void* stream);
int aprnet_upsample_fwd_bf16g(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int C, uint16_t* y, int64_t ldy,
                              void* stream);
int aprnet_conv111_fwd_bf16g(const aprnet_plan*, int level_delta, const uint16_t* x, int64_t ldx, int Cin, const float* w, int S,
                             int Cout, const float* bias, int relu, uint16_t* y, int64_t ldy, int y_grouped, void* stream);
/* largest Cin that aprnet_conv111_fwd_bf16g takes (256): callers that choose between the grouped and the plane
 * operators ask before they start a network (no counterpart in the reference) */
int aprnet_conv111_g8_max_cin(void);
int aprnet_conv_fwd_fused_bf16l(const aprnet_plan*, int level_delta, int kz, int kx, int ky, const uint16_t* x, int64_t ldx, int Cin,
                                int x_grouped, const float* w, int S_exp, int Cout, const float* bias, uint16_t* y, int64_t ldy,
                                int y_grouped, uint16_t* tree_ws, int64_t ld_tree, const aprnet_conv_fusion* fusion, void* stream);
/* The last stencil convolution of a network together with the 1x1x1 convolution that follows it (the head of the
 * APR-UNet: apr_models/apr_models/unet/unet_model.py:75-79, applied at :94 to the last UpConv block's output): x (and fusion->x2) grouped,
 * Cout <= 16; the layer's result - after bias and fusion->relu, rounded to bfloat16 as aprnet_conv_fwd_fused_bf16l
 * would store it - is not written; out [head_C][ldo] planes = Convolution<1,1,1>::forward of it with
 * head_w [head_S][head_C][Cout] and head_bias [head_C] (or NULL), head_C <= 4, fp32 products and sums.  Saves one
 * write and one read of the 16-channel tensor at the network's full resolution. */
int aprnet_conv_fwd_head_bf16g(const aprnet_plan*, int level_delta, int kz, int kx, int ky, const uint16_t* x, int64_t ldx, int Cin,
                               const float* w, int S_exp, int Cout, const float* bias, uint16_t* tree_ws, int64_t ld_tree,
                               const aprnet_conv_fusion* fusion, const float* head_w, int head_S, int head_C,
                               const float* head_bias, uint16_t* out, int64_t ldo, void* stream);

/* Label and coordinate utilities of the StarDist networks (pyapr/aprnet/src/utils.hpp:86-333; CPU loops in the
 * reference, device kernels here).  Particle order = feature order at level_delta.  Images are dense device arrays
 * [zn][xn][yn] with the dimensions of the APR's finest level.
 *   particle_coords   get_particle_coords (utils.hpp:222-267): coords [N_d][3] = (z, x, y) cell centres in pixels.
 *   sample_image_max  sample_image (utils.hpp:270-333): parts [N_d] = maximum of img over each particle's cell.
 *   labels_to_dist    labels_to_dist_cpp (utils.hpp:86-219): dist [N_d][n_rays], left untouched (caller zeroes it)
 *                     where the particle's centre carries label 0 or lies outside the image.  dzs / dxs / dys:
 *                     device arrays [n_rays] of the ray steps.  max_steps bounds the walk along a ray (the
 *                     reference walks until the ray leaves its object, which never ends for a zero step). */
int aprnet_particle_coords(const aprnet_plan*, int level_delta, float* coords, void* stream);
int aprnet_sample_image_max_f32(const aprnet_plan*, int level_delta, const float* img, int zn, int xn, int yn, float* parts,
                                void* stream);
int aprnet_labels_to_dist_u8(const aprnet_plan*, int level_delta, const uint8_t* img, int zn, int xn, int yn, const float* dzs,
                             const float* dxs, const float* dys, int n_rays, int max_steps, float* dist, void* stream);
int aprnet_labels_to_dist_u16(const aprnet_plan*, int level_delta, const uint16_t* img, int zn, int xn, int yn, const float* dzs,
                              const float* dxs, const float* dys, int n_rays, int max_steps, float* dist, void* stream);
int aprnet_labels_to_dist_u32(const aprnet_plan*, int level_delta, const uint32_t* img, int zn, int xn, int yn, const float* dzs,
                              const float* dxs, const float* dys, int n_rays, int max_steps, float* dist, void* stream);
int aprnet_labels_to_dist_u64(const aprnet_plan*, int level_delta, const uint64_t* img, int zn, int xn, int yn, const float* dzs,
                              const float* dxs, const float* dys, int n_rays, int max_steps, float* dist, void* stream);

/* Normalisation over the particle axis and the ReLU after it: the torch.nn.BatchNorm1d / torch.nn.GroupNorm +
 * activation that follow every convolution of the networks (apr_models/unet/unet_parts.py:17-26; library calls on
 * [batch, channels, particles] tensors in the reference, MIOpen / ATen kernels on a GPU).  The kernels work on
 * rows: row r = one (batch item, channel) line of n elements at x + r * ldx.  The per-row results are joined into
 * per-channel (BatchNorm) or per-group (GroupNorm) statistics - a few values per row - by aprnet_norm_coeffs_*,
 * which hand per-row coefficients back.  rows <= 65535, n > 0.  work: aprnet_norm_work_elems(rows) floats of scratch.
 *   row_moments     mean[r], m2[r] = mean and sum of squared deviations of row r (fp64 results).
 *   norm_apply      y = (x - mean[r]) * scale[r] + shift[r], then max(., 0) if relu != 0.
 *   norm_bwd_sums   sum_g[r] = sum g, sum_gx[r] = sum g * xhat with xhat = (x - mean[r]) * rstd[r] and
 *                   g = gy, or gy where y > 0 and 0 elsewhere when y (the forward output) is given.
 *   norm_bwd_apply  gx = a[r] * g + b[r] * xhat + c[r].
 * Sums are taken in a fixed order (fp32 per thread and block, fp64 across blocks): results repeat bit for bit. */
int64_t aprnet_norm_work_elems(int64_t rows);
/* The join between the row kernels, one launch each way (the arithmetic of torch.nn.BatchNorm1d when groups == 0 -
 * a channel's rows over the batch share statistics - and of torch.nn.GroupNorm(groups, C) otherwise; biased
 * variance).  Arrays are [B * C] per row unless noted; gamma / beta [C] or NULL.
 *   coeffs_fwd  from row_mean / row_m2 (row_moments), or from given_mean / given_var [C] (BatchNorm in eval mode)
 *               when those are not NULL: mean32, rstd32, scale32 = gamma * rstd, shift32 = beta for norm_apply, and
 *               the statistics used, set_mean / set_var ([C], or [B * groups]; not written with given statistics).
 *   coeffs_bwd  from the sums of norm_bwd_sums: a, b, c for norm_bwd_apply (b = c = 0 when own_stats == 0, i.e. the
 *               statistics did not depend on the input) and grad_gamma / grad_beta [C] (each may be NULL). */
int aprnet_norm_coeffs_fwd(int B, int C, int groups, int64_t n, double eps, const double* row_mean, const double* row_m2,
                           const float* given_mean, const float* given_var, const float* gamma, const float* beta,
                           float* mean32, float* rstd32, float* scale32, float* shift32, float* set_mean, float* set_var,
                           void* stream);
int aprnet_norm_coeffs_bwd(int B, int C, int groups, int64_t n, int own_stats, const double* sum_g, const double* sum_gx,
                           const float* gamma, const float* rstd32, float* a, float* b, float* c, float* grad_gamma,
                           float* grad_beta, void* stream);
int aprnet_row_moments_f32(const float* x, int64_t ldx, int64_t rows, int64_t n, double* mean, double* m2, float* work, void* stream);
int aprnet_row_moments_bf16(const uint16_t* x, int64_t ldx, int64_t rows, int64_t n, double* mean, double* m2, float* work, void* stream);
int aprnet_norm_apply_f32(const float* x, int64_t ldx, int64_t rows, int64_t n, const float* mean, const float* scale,
                          const float* shift, int relu, float* y, int64_t ldy, void* stream);
int aprnet_norm_apply_bf16(const uint16_t* x, int64_t ldx, int64_t rows, int64_t n, const float* mean, const float* scale,
                           const float* shift, int relu, uint16_t* y, int64_t ldy, void* stream);
int aprnet_norm_bwd_sums_f32(const float* gy, int64_t ldg, const float* x, int64_t ldx, const float* y, int64_t ldy, int64_t rows,
                             int64_t n, const float* mean, const float* rstd, double* sum_g, double* sum_gx, float* work,
                             void* stream);
int aprnet_norm_bwd_sums_bf16(const uint16_t* gy, int64_t ldg, const uint16_t* x, int64_t ldx, const uint16_t* y, int64_t ldy,
                              int64_t rows, int64_t n, const float* mean, const float* rstd, double* sum_g, double* sum_gx,
                              float* work, void* stream);
int aprnet_norm_bwd_apply_f32(const float* gy, int64_t ldg, const float* x, int64_t ldx, const float* y, int64_t ldy, int64_t rows,
                              int64_t n, const float* mean, const float* rstd, const float* a, const float* b, const float* c,
                              float* gx, int64_t ldo, void* stream);
int aprnet_norm_bwd_apply_bf16(const uint16_t* gy, int64_t ldg, const uint16_t* x, int64_t ldx, const uint16_t* y, int64_t ldy,
                               int64_t rows, int64_t n, const float* mean, const float* rstd, const float* a, const float* b,
                               const float* c, uint16_t* gx, int64_t ldo, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* APRNET_HIP_H */
