"""The entry point that allocates nothing: aprnet_channel_sum_static_f32 keeps the block partials of the bias-gradient
sum in a device array of the library.  Checked against aprnet_channel_sum_f32 (same kernels, caller work space):
bit-equal, on two calls in a row, the second with a smaller input (the array keeps the first call's partials)."""
import ctypes as C

import pytest
import torch

from pyapr import _native

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _both(lib, x, accumulate_into=None):
    c, n = x.shape
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    work = torch.empty(lib.aprnet_channel_sum_work_elems(c), dtype=torch.float32, device=DEV)
    ref = torch.zeros(c, device=DEV) if accumulate_into is None else accumulate_into.clone()
    got = ref.clone()
    acc = 0 if accumulate_into is None else 1
    assert lib.aprnet_channel_sum_f32(C.c_void_p(x.data_ptr()), n, c, n, C.c_void_p(ref.data_ptr()), acc,
                                      C.c_void_p(work.data_ptr()), st) == 0
    assert lib.aprnet_channel_sum_static_f32(C.c_void_p(x.data_ptr()), n, c, n, C.c_void_p(got.data_ptr()), acc, st) == 0, \
        lib.aprnet_last_error().decode()
    torch.cuda.synchronize()
    return got, ref


def test_static_channel_sum_matches_the_work_space_entry_point():
    lib = _native.hip()
    g = torch.Generator().manual_seed(0)
    big = torch.randn(48, 300_007, generator=g).to(DEV)
    got, ref = _both(lib, big)
    assert torch.equal(got, ref)
    torch.testing.assert_close(got.cpu().double(), big.cpu().double().sum(dim=1), rtol=1e-5, atol=1e-2)
    # second call, smaller in both directions: stale partials of the first call must not leak into it
    small = torch.randn(5, 1_001, generator=g).to(DEV)
    got2, ref2 = _both(lib, small)
    assert torch.equal(got2, ref2)
    torch.testing.assert_close(got2.cpu().double(), small.cpu().double().sum(dim=1), rtol=1e-5, atol=1e-3)
    # accumulate flag (batch items after the first) and the channel limit
    got3, ref3 = _both(lib, small, accumulate_into=got2)
    assert torch.equal(got3, ref3)
    cmax = lib.aprnet_channel_sum_static_max_channels()
    too_wide = torch.zeros(cmax + 1, 8, device=DEV)
    out = torch.zeros(cmax + 1, device=DEV)
    rc = lib.aprnet_channel_sum_static_f32(C.c_void_p(too_wide.data_ptr()), 8, cmax + 1, 8, C.c_void_p(out.data_ptr()), 0, None)
    assert rc == -4 and "channels" in lib.aprnet_last_error().decode()
