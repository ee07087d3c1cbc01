"""CPU-side checks of the drop-in boundary: the C-ABI library loads without a GPU and exports every
symbol that include/aprnet_hip.h declares; the Python host layer mirrors the reference's module API and
refuses to run without device tensors (no CPU fallback)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aprnet_hip.h")
LIB = os.path.join(ROOT, "apr-cnn_amd", "csrc", "libaprnet_hip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b(aprnet_[a-z0-9_]+)\s*\(", text))
    macro = re.search(r"#define APRNET_DECL\(T, SFX\)(.*?)\n\nAPRNET_DECL", text, flags=re.S).group(1)
    for base in re.findall(r"\b(aprnet_[a-z0-9_]+_)##SFX", macro):
        for sfx in ("f32", "f64"):
            names.add(base + sfx)
    return sorted(n for n in names if not n.endswith("_"))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    names = declared_symbols()
    assert len(names) >= 39
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in aprnet_hip.h but not exported: {missing}"


def test_module_api_mirrors_reference():
    from pyapr import aprnet
    from pyapr.aprnet import cuda
    # constructor signature / parameter names / layouts (conv.py:154-166, cuda/conv.py:66-79)
    m = aprnet.APRConv(3, 5, nstencils=2, kernel_size=(1, 5, 5), bias=True)
    assert tuple(m.weight.shape) == (3, 2, 5, 1, 5, 5) and tuple(m.bias.shape) == (5,)
    assert set(m.state_dict()) == {"weight", "bias"}
    mc = cuda.APRConv(3, 5, nstencils=2, kernel_size=(3, 3, 3), bias=False)
    assert tuple(mc.weight.shape) == (2, 5, 3, 3, 3, 3) and mc.bias is None
    assert set(mc.state_dict()) == {"weight"}
    # kaiming_uniform_(a=sqrt(5)) bound: sqrt(6 / ((1 + 5) * fan_in)) with fan_in = size(1) * receptive field
    fan_in = mc.weight.shape[1] * 27
    assert float(mc.weight.abs().max()) <= (1.0 / fan_in) ** 0.5 + 1e-6
    assert aprnet.MaxPool().increment_level_deltas is True
    assert aprnet.UpSampleConst().decrement_level_deltas is True
    for name in ("APRConv", "MaxPool", "UpSampleConst", "Reconstruct", "SampleParticles"):
        assert hasattr(cuda, name)
    for name in ("number_particles", "number_parts", "number_particles_after_pooling", "number_particles_after_upsampling"):
        assert hasattr(aprnet.utils, name)


def test_no_cpu_fallback():
    """Operators refuse host tensors (CHECK_CUDA, cuda/src/common.hpp:14) instead of computing on the CPU."""
    import apr_cases
    from pyapr import aprnet
    apr = apr_cases.get("3d_a")
    n = aprnet.utils.number_particles(apr, 0)
    x = torch.zeros(1, 1, n)
    ld = torch.zeros(1, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        aprnet.MaxPool()(x, [apr], ld)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        aprnet.cuda.APRConv(1, 1, kernel_size=(1, 1, 1))(x, [apr], ld)


def test_number_particles_helpers():
    import apr_cases
    from oracle import oracle
    from pyapr import aprnet
    for name in ("3d_a", "2d_b", "1d_a", "3d_s"):
        apr = apr_cases.get(name)
        for d in range(apr.level_max() - 1):
            assert aprnet.utils.number_particles(apr, d) == oracle.number_parts(apr, d)
            assert aprnet.utils.number_particles_after_pooling(apr, d) == oracle.number_parts(apr, d + 1)
        assert aprnet.utils.number_particles(apr, 0) == apr.total_number_particles()


def test_apr_state_roundtrip():
    """The serialisable state is the one of BindAPR.hpp:72-90; level_xz_vec is recomputed from the dims."""
    import numpy as np
    import apr_cases
    from pyapr import APR
    apr = apr_cases.get("3d_b")
    oy, ox, oz, _params, xz, y, txz, ty = apr.get_state()
    back = APR.from_state((oy, ox, oz), xz, y, txz, ty)
    for a, b in ((apr.iterator(), back.iterator()), (apr.tree_iterator(), back.tree_iterator())):
        assert np.array_equal(a.level_xz_vec, b.level_xz_vec) and np.array_equal(a.xz_end_vec, b.xz_end_vec)
        assert np.array_equal(a.y_vec, b.y_vec) and a.level_min() == b.level_min() and a.level_max() == b.level_max()


def test_model_parameter_names_mirror_reference():
    """state_dict keys of the networks are those of the reference's module trees (unet_parts.py:6-83,
    hybrid_unet_parts.py:9-128, unet_model.py / hybrid_model.py), so checkpoints are interchangeable."""
    from apr_models.unet import APRUNet, HybridAPRUNet, APRStardistUNet, HybridStardistUNet
    keys = set(APRUNet(1, 2, depth=1, n_filters_base=4).state_dict())
    assert {"encoder.0.blocks.0.conv.weight", "encoder.0.blocks.1.norm.weight", "encoder.1.conv.blocks.0.conv.weight",
            "decoder.0.reduce_ch.conv.weight", "decoder.0.conv.blocks.1.norm.bias", "head.weight", "head.bias"} <= keys
    hyb = HybridAPRUNet(1, 2, depth=3, apr_depth=1, n_filters_base=4)
    keys = set(hyb.state_dict())
    assert {"encoder.1.conv.blocks.0.conv.weight",            # DownConv (particles)
            "encoder.2.conv.blocks.0.conv.weight",            # TransitionDownConv (dense Conv3d)
            "encoder.3.conv.blocks.1.norm.weight",            # PixelDownConv
            "decoder.0.reduce_ch.conv.weight",                # PixelUpConv
            "decoder.1.reduce_ch.conv.weight", "decoder.1.conv.blocks.0.conv.weight",      # TransitionUpConv
            "decoder.2.reduce_ch.conv.weight", "head.weight"} <= keys
    for net in (APRStardistUNet(1, 4, depth=1, n_filters_base=4), HybridStardistUNet(1, 4, depth=2, apr_depth=1, n_filters_base=4)):
        assert {"output_prob.conv.weight", "output_dist.weight", "output_dist.bias"} <= set(net.state_dict())
    sd = hyb.state_dict()
    assert sd["encoder.2.conv.blocks.0.conv.weight"].dim() == 5       # nn.Conv3d [Cout, Cin, kz, kx, ky]
    assert sd["decoder.1.conv.blocks.0.conv.weight"].dim() == 6       # APRConv [S, Cout, Cin, kz, kx, ky]
    assert tuple(sd["decoder.1.conv.blocks.0.conv.weight"].shape[1:3]) == (8, 16)      # reads skip + upsampled


def test_plan_create_refuses_damaged_access_arrays():
    """Access arrays read from a file are validated on the host before any device work: a damaged state is
    APRNET_ERR_INVALID_ARGUMENT (-1) with a message naming the violation, not an out-of-range access on the GPU.
    Runs without a GPU: validation comes before the first HIP call."""
    import ctypes as C
    import numpy as np
    import apr_cases
    from pyapr import APR, _native
    lib = _native.hip()
    good = apr_cases.get("3d_a")
    oy, ox, oz, _params, xz, y, txz, ty = good.get_state()

    def create(xz_, y_, txz_, ty_, drop_y=False):
        apr = APR.from_state((oy, ox, oz), np.array(xz_), np.array(y_), np.array(txz_), np.array(ty_))
        a, t = apr._desc(apr.iterator()), apr._desc(apr.tree_iterator())
        if drop_y:
            a.y_vec = None
        h = C.c_void_p()
        rc = lib.aprnet_plan_create(C.byref(a), C.byref(t), 0, C.byref(h))
        msg = lib.aprnet_last_error().decode()
        if rc == 0:
            lib.aprnet_plan_destroy(h)
        return rc, msg

    # a row with two or more particles, to break the order inside it
    rows = np.flatnonzero(np.diff(xz.astype(np.int64)) >= 2)
    b = int(xz[rows[0]])
    y_swapped = y.copy(); y_swapped[b], y_swapped[b + 1] = y[b + 1], y[b]
    rc, msg = create(xz, y_swapped, txz, ty)
    assert rc == -1 and "ascend" in msg
    y_big = y.copy(); y_big[b + 1] = 65535
    rc, msg = create(xz, y_big, txz, ty)
    assert rc == -1 and "y_num" in msg
    xz_bad = xz.copy(); xz_bad[rows[0] + 1] = xz_bad[rows[0]] - 1 if xz_bad[rows[0]] > 0 else xz_bad[-1] + 5
    rc, msg = create(xz_bad, y, txz, ty)
    assert rc == -1 and ("xz_end_vec" in msg or "y_vec" in msg)       # a moved row end also mis-slices y
    xz_over = xz.copy(); xz_over[len(xz) // 2] = xz[-1] + 7
    rc, msg = create(xz_over, y, txz, ty)
    assert rc == -1 and "xz_end_vec" in msg
    ty_bad = ty.copy()
    trows = np.flatnonzero(np.diff(txz.astype(np.int64)) >= 2)
    tb = int(txz[trows[0]]); ty_bad[tb + 1] = ty_bad[tb]
    rc, msg = create(xz, y, txz, ty_bad)
    assert rc == -1 and "ascend" in msg
    rc, msg = create(xz, y, txz, ty, drop_y=True)
    assert rc == -1 and "y_vec" in msg


def test_compiled_binding_exposes_the_reference_names():
    """The pybind11 module builds in-tree, imports without a GPU and registers the native function names of
    wrappers/pythonBind.cpp:144-182, wrap_conv.hpp:12-49, wrap_pool.hpp:14-15, wrap_upsample.hpp:14-15 and
    utils.hpp:340-380 (the operator part)."""
    import _pyaprwrapper
    m = _pyaprwrapper.aprnet
    cuda = ["maxpool_forward_cuda", "maxpool_backward_cuda", "conv111_forward", "conv111_backward", "conv333_forward",
            "conv333_backward", "upsample_const_forward", "upsample_const_backward", "restrict_kernel333_forward",
            "restrict_kernel333_backward", "reconstruct_forward", "reconstruct_backward", "sample_particles_forward",
            "sample_particles_backward"]
    conv = [f"convolve{k}_{d}" for k in ("111", "333", "133", "555", "155") for d in ("forward", "backward")]
    conv += [f"restrict_kernel{k}_{d}" for k in ("333", "133", "555", "155") for d in ("forward", "backward")]
    for mod, names in ((m.cuda, cuda), (m.conv, conv), (m.pool, ["maxpool_forward", "maxpool_backward"]),
                       (m.upsample, ["upsample_const_forward", "upsample_const_backward"]),
                       (m.utils, ["number_particles", "number_parts", "number_particles_after_pooling",
                                  "number_particles_after_upsampling"])):
        missing = [n for n in names if not hasattr(mod, n)]
        assert not missing, missing
    import apr_cases
    apr = apr_cases.get("3d_a")
    assert m.utils.number_particles(apr, 0) == apr.total_number_particles()
    with pytest.raises(RuntimeError, match="CUDA tensor"):          # CHECK_INPUT, cuda/src/common.hpp:14-16
        m.cuda.conv333_forward([apr], torch.zeros(1, 1, 4), torch.zeros(1, 1, 1, 3, 3, 3), torch.zeros(1, dtype=torch.int32))


def test_kernel_selection_switch_answers_only_in_a_testing_process():
    """aprnet_set_conv_path is process-wide, so it is shut unless the process asked for it: without APRNET_TESTING=1
    in the environment every value is refused (and nothing changes), with it the documented values are taken and
    unknown ones are refused.  Checked in fresh processes, because the flag is read once."""
    import subprocess
    import sys
    code = ("import ctypes, sys; lib = ctypes.CDLL(sys.argv[1]); "
            "print(lib.aprnet_set_conv_path(1), lib.aprnet_set_conv_path(0), lib.aprnet_set_conv_path(17), "
            "lib.aprnet_set_conv_path(16), lib.aprnet_set_conv_path(99))")
    def run(env_value):
        env = {k: v for k, v in os.environ.items() if k != "APRNET_TESTING"}
        if env_value is not None:
            env["APRNET_TESTING"] = env_value
        out = subprocess.run([sys.executable, "-c", code, LIB], env=env, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        return [int(v) for v in out.stdout.split()]
    for off in (None, "0", ""):
        assert all(rc != 0 for rc in run(off))
    on = run("1")
    assert on[:4] == [0, 0, 0, 0] and on[4] != 0
