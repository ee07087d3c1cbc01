"""ctypes bindings to the two native libraries of this package.

* ``libaprcore.so``    host-only C++/OpenMP: APR access-structure builder, synthetic volumes.
* ``libaprnet_hip.so`` the C-ABI of the HIP operators (declared in ``include/aprnet_hip.h``).

Both are built in-tree under ``csrc/`` (``python csrc/build.py``).  Nothing here falls back to a
Python or CPU implementation: a missing library raises ``ImportError`` naming the build command.
"""
import ctypes as C
import os

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")

_core = None
_hip = None


def _load(name):
    # APRNET_LIB_DIR points at an alternative build of the two libraries (kernel experiments)
    path = os.path.join(os.environ.get("APRNET_LIB_DIR", _CSRC), name)
    if not os.path.exists(path):
        raise ImportError(
            f"{name} is not built: run `python {os.path.join(_CSRC, 'build.py')}` "
            f"(hipcc --offload-arch=gfx950) first; there is no fallback path")
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


def core():
    """libaprcore.so with argtypes set."""
    global _core
    if _core is not None:
        return _core
    lib = _load("libaprcore.so")
    vp, i32, i64, u64, f32 = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_float
    lib.aprcore_last_error.restype = C.c_char_p
    lib.aprcore_create.restype = vp
    lib.aprcore_create.argtypes = [i32, i32, i32]
    lib.aprcore_destroy.argtypes = [vp]
    lib.aprcore_level_max.argtypes = [vp]
    lib.aprcore_level_dims.argtypes = [vp, i32, vp]
    lib.aprcore_build_from_levels.argtypes = [vp, vp]
    lib.aprcore_access_info.argtypes = [vp, i32, vp]
    lib.aprcore_access_copy.argtypes = [vp, i32, vp, vp, vp, vp, vp, vp]
    lib.aprcore_level_field_u16.argtypes = [vp, vp, f32, f32, f32, f32, f32, vp]
    lib.aprcore_sample_mean_u16.argtypes = [vp, vp, vp]
    lib.aprcore_synth_volume_u16.argtypes = [vp, i32, i32, i32, u64, i32, i32, f32, f32, i32, f32, f32,
                                             f32, f32, i32]
    _core = lib
    return lib


class AccessDesc(C.Structure):
    """Mirror of ``aprnet_access_desc`` in include/aprnet_hip.h (all pointers are host pointers)."""
    _fields_ = [
        ("level_min", C.c_int32), ("level_max", C.c_int32),
        ("z_num", C.c_void_p), ("x_num", C.c_void_p), ("y_num", C.c_void_p),
        ("level_xz_vec", C.c_void_p), ("xz_end_vec", C.c_void_p), ("y_vec", C.c_void_p),
        ("n_rows", C.c_uint64), ("n_particles", C.c_uint64),
    ]


def hip():
    """libaprnet_hip.so with argtypes set (loads without a GPU; calls need one)."""
    global _hip
    if _hip is not None:
        return _hip
    lib = _load("libaprnet_hip.so")
    vp, i32, i64 = C.c_void_p, C.c_int, C.c_int64
    P = C.POINTER
    lib.aprnet_last_error.restype = C.c_char_p
    lib.aprnet_plan_create.argtypes = [P(AccessDesc), P(AccessDesc), i32, P(vp)]
    lib.aprnet_plan_destroy.argtypes = [vp]
    for fn in ("aprnet_number_parts", "aprnet_tree_offset", "aprnet_tree_parts"):
        getattr(lib, fn).restype = i64
        getattr(lib, fn).argtypes = [vp, i32]
    lib.aprnet_plan_children.argtypes = [vp, vp]
    lib.aprnet_plan_reserve.argtypes = [vp, i64, vp]
    lib.aprnet_profile_enable.argtypes = [i32]
    lib.aprnet_set_conv_path.argtypes = [i32]
    lib.aprnet_profile_last_ms.restype = C.c_float
    for t in ("f32", "f64"):
        getattr(lib, f"aprnet_fill_tree_mean_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_fill_tree_mean_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_channel_sum_{t}").argtypes = [vp, i64, i32, i64, vp, i32, vp, vp]
        getattr(lib, f"aprnet_conv_fwd_{t}").argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp,
                                                         vp, i64, vp, i64, vp]
        getattr(lib, f"aprnet_conv_bwd_{t}").argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32,
                                                         vp, i64, vp, i64, vp, vp, i64, vp, i64, vp]
        getattr(lib, f"aprnet_conv111_fwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i32, i32, vp, vp, i64, vp]
        getattr(lib, f"aprnet_conv111_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i32, i32, vp, i64,
                                                            vp, i64, vp, vp]
        getattr(lib, f"aprnet_maxpool_fwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp, i64, vp]
        getattr(lib, f"aprnet_maxpool_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp, i64, vp]
        getattr(lib, f"aprnet_upsample_fwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_upsample_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_restrict_kernel_fwd_{t}").argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp]
        getattr(lib, f"aprnet_restrict_kernel_bwd_{t}").argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp]
        getattr(lib, f"aprnet_reconstruct_fwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_reconstruct_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_sample_particles_fwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
        getattr(lib, f"aprnet_sample_particles_bwd_{t}").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    # bfloat16 features: forward operators of the network, backward of pool / upsample / tree fill
    lib.aprnet_conv_fwd_bf16.argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp, vp, i64, vp, i64, vp]
    lib.aprnet_particle_coords.argtypes = [vp, i32, vp, vp]
    lib.aprnet_sample_image_max_f32.argtypes = [vp, i32, vp, i32, i32, i32, vp, vp]
    for t in ("u8", "u16", "u32", "u64"):     # plan, d, img, zn, xn, yn, dzs, dxs, dys, n_rays, max_steps, dist, stream
        getattr(lib, f"aprnet_labels_to_dist_{t}").argtypes = [vp, i32, vp, i32, i32, i32, vp, vp, vp, i32, i32, vp, vp]
    f64 = C.c_double
    lib.aprnet_norm_coeffs_fwd.argtypes = [i32, i32, i32, i64, f64, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.aprnet_norm_coeffs_bwd.argtypes = [i32, i32, i32, i64, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.aprnet_norm_work_elems.argtypes = [i64]
    lib.aprnet_norm_work_elems.restype = i64
    for t in ("f32", "bf16"):
        getattr(lib, f"aprnet_row_moments_{t}").argtypes = [vp, i64, i64, i64, vp, vp, vp, vp]
        getattr(lib, f"aprnet_norm_apply_{t}").argtypes = [vp, i64, i64, i64, vp, vp, vp, i32, vp, i64, vp]
        getattr(lib, f"aprnet_norm_bwd_sums_{t}").argtypes = [vp, i64, vp, i64, vp, i64, i64, i64, vp, vp, vp, vp, vp, vp]
        getattr(lib, f"aprnet_norm_bwd_apply_{t}").argtypes = [vp, i64, vp, i64, vp, i64, i64, i64, vp, vp, vp, vp, vp, vp, i64, vp]
    for t in ("f32", "f64", "bf16"):      # ..., tree_ws, ld_tree, const aprnet_conv_fusion*, stream
        getattr(lib, f"aprnet_conv_fwd_fused_{t}").argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp, vp, i64,
                                                                vp, i64, vp, vp]
    lib.aprnet_conv111_fwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i32, i32, vp, vp, i64, vp]
    lib.aprnet_conv111_bwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i32, i32, vp, i64, vp, i64, vp, vp]
    lib.aprnet_fill_tree_mean_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_fill_tree_mean_bwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_maxpool_fwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp, i64, vp]
    lib.aprnet_maxpool_bwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp, i64, vp]
    lib.aprnet_upsample_fwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_upsample_bwd_bf16.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    for op in ("reconstruct_fwd", "reconstruct_bwd", "sample_particles_fwd", "sample_particles_bwd"):
        getattr(lib, f"aprnet_{op}_bf16").argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_channel_sum_work_elems.argtypes = [i32]
    lib.aprnet_channel_sum_static_f32.argtypes = [vp, i64, i32, i64, vp, i32, vp]
    lib.aprnet_channel_sum_bf16.argtypes = [vp, i64, i32, i64, vp, i32, vp, vp]
    lib.aprnet_conv_bwd_bf16.argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp, i64, vp, i64, vp,
                                         vp, i64, vp, i64, vp, i64, vp]
    # bfloat16 features grouped by eight channels
    lib.aprnet_regroup8_bf16.argtypes = [vp, i64, i32, i64, vp, i64, vp]
    lib.aprnet_ungroup8_bf16.argtypes = [vp, i64, i32, i64, vp, i64, vp]
    lib.aprnet_fill_tree_mean_bf16g.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_maxpool_fwd_bf16g.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_upsample_fwd_bf16g.argtypes = [vp, i32, vp, i64, i32, vp, i64, vp]
    lib.aprnet_conv111_fwd_bf16g.argtypes = [vp, i32, vp, i64, i32, vp, i32, i32, vp, i32, vp, i64, i32, vp]
    lib.aprnet_conv_fwd_fused_bf16l.argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, i32, vp, i32, i32, vp, vp, i64, i32,
                                                vp, i64, vp, vp]
    lib.aprnet_conv_fwd_head_bf16g.argtypes = [vp, i32, i32, i32, i32, vp, i64, i32, vp, i32, i32, vp, vp, i64, vp,
                                               vp, i32, i32, vp, vp, i64, vp]
    _hip = lib
    return lib
