"""Plan housekeeping around HIP graphs: the scratch buffer of a plan never moves under a captured graph, and what
would have to allocate during a capture is an error code instead of a failed capture."""
import pytest
import torch

import apr_cases
from pyapr.aprnet import _ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _weights(levels, cout, cin, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(levels, cout, cin, 3, 3, 3, generator=g) * 0.2).to(DEV)


def test_graph_replays_correctly_after_the_scratch_buffer_grew():
    """capture a small layer -> run a wider layer eagerly (its packed weights need a larger scratch buffer) -> the
    graph still replays into memory it owns and reproduces the eager result bit for bit."""
    apr = apr_cases.random_apr((33, 29, 37), 21, density=0.02)
    n = apr.total_number_particles()
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator().manual_seed(0)
    x_static = torch.randn(1, 4, n, generator=g).to(DEV)
    w_small = _weights(levels, 4, 4, 1)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            _ops.conv_forward([apr], x_static, w_small, ld)          # builds the lists, sizes the scratch for 4 -> 4
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = _ops.conv_forward([apr], x_static, w_small, ld)
        # a much wider layer on the same plan: the scratch buffer has to grow
        x_wide = torch.randn(1, 48, n, generator=g).to(DEV)
        w_wide = _weights(levels, 64, 48, 2)
        y_wide = _ops.conv_forward([apr], x_wide, w_wide, ld)
        torch.cuda.synchronize()
        assert torch.isfinite(y_wide).all()
        for k in range(3):
            x_new = torch.randn(1, 4, n, generator=g).to(DEV)
            eager = _ops.conv_forward([apr], x_new, w_small, ld)
            torch.cuda.synchronize()
            x_static.copy_(x_new)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_static, eager), f"replay {k}"
            _ops.conv_forward([apr], x_wide, w_wide, ld)             # the wide layer keeps using the new buffer
            torch.cuda.synchronize()


def test_growth_and_first_use_during_capture_are_refused():
    """Under capture the first convolution of a plan (tile and window lists) and a layer that needs a larger scratch
    buffer return APRNET_ERR_UNSUPPORTED (RuntimeError here) before anything is launched; after
    aprnet_plan_reserve the same layer captures."""
    from pyapr import _native
    apr = apr_cases.random_apr((33, 29, 37), 22, density=0.02)
    apr.init_cuda()
    n = apr.total_number_particles()
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator().manual_seed(0)
    x4 = torch.randn(1, 4, n, generator=g).to(DEV)
    x48 = torch.randn(1, 48, n, generator=g).to(DEV)
    w_small, w_wide = _weights(levels, 4, 4, 1), _weights(levels, 64, 48, 2)
    with torch.no_grad():
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            with pytest.raises(RuntimeError, match="captur"):
                _ops.conv_forward([apr], x4, w_small, ld)            # nothing built yet
        eager_small = _ops.conv_forward([apr], x4, w_small, ld)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            with pytest.raises(RuntimeError, match="captur"):
                _ops.conv_forward([apr], x48, w_wide, ld)            # lists are there, the scratch is too small
        lib = _native.hip()
        assert lib.aprnet_plan_reserve(apr.plan(0), 64 << 20, None) == 0
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_wide = _ops.conv_forward([apr], x48, w_wide, ld)
        graph.replay()
        torch.cuda.synchronize()
        eager_wide = _ops.conv_forward([apr], x48, w_wide, ld)
        assert torch.equal(y_wide, eager_wide)
        assert torch.equal(_ops.conv_forward([apr], x4, w_small, ld), eager_small)
