"""sub1_moe_grouped_prepared_static: the expert-layer launch whose scratch
memory (control words and h) is a static device array instead of a workspace
argument, for callers that cannot allocate.  Called through the C ABI, its
output must equal sub1_moe_grouped_prepared's bit for bit, on two calls in a
row, the second on a smaller batch (the array keeps the first call's
contents); batches beyond the array are refused."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import sub1_oracle as so
from test_gpu_parity import bf16_dev, bits_host, small_stack

pytestmark = pytest.mark.gpu


def test_static_scratch_launch_equals_workspace_launch(oracle):
    from qmoe_amd import _lib, sub1
    assert torch.cuda.is_available() and sub1.DEC
    lib = _lib.load()
    _lib.check(lib.sub1_init())
    experts, d_model, d_ff = 4, 768, 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=1500)
    prep = stack.prepare()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def both(route, seed):
        tokens = len(route)
        xs = np.stack([so.synthetic_activation(d_model, seed + i) for i in range(tokens)])
        x = bf16_dev(xs)
        te = torch.tensor(route, dtype=torch.int32, device='cuda')
        want = prep.forward(x, te)                       # sub1_moe_grouped_prepared
        got = torch.full_like(x, 7.0)
        _lib.check(lib.sub1_moe_grouped_prepared_static(
            ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(), got.data_ptr(), tokens, stream))
        torch.cuda.synchronize()
        return xs, bits_host(got), bits_host(want)

    # the first call: 40 tokens, some dropped, one with an expert that does not exist
    route = [(3 * i) % experts for i in range(40)]
    route[5], route[17], route[30] = -1, experts + 1, -1
    xs, got, want = both(route, 1600)
    assert np.array_equal(got, want)
    for i in (0, 7, 39):
        ref, _ = oracle.expert_ffn(wi[route[i]], wo[route[i]], xs[i], order=2)
        assert np.array_equal(got[i], ref)
    for i in (5, 17, 30):
        assert np.array_equal(got[i], xs[i])
    # the second, smaller, on the same array
    route = [2, 0, 3]
    xs, got, want = both(route, 1700)
    assert np.array_equal(got, want)
    for i, e in enumerate(route):
        ref, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)
        assert np.array_equal(got[i], ref)
    # and a larger one again: the small call's h must not have landed on the
    # words that this one's workgroups count with
    route = [(5 * i + 1) % experts for i in range(40)]
    xs, got, want = both(route, 1800)
    assert np.array_equal(got, want)
    for i in (0, 21, 39):
        ref, _ = oracle.expert_ffn(wi[route[i]], wo[route[i]], xs[i], order=2)
        assert np.array_equal(got[i], ref)
    _lib.check_faults()

    # more scratch than the array holds: refused, with the size in the message
    tokens = 200
    assert lib.sub1_moe_workspace_bytes(tokens, d_ff) > (1 << 20)
    x = torch.zeros((tokens, d_model), dtype=torch.bfloat16, device='cuda')
    te = torch.zeros(tokens, dtype=torch.int32, device='cuda')
    rc = lib.sub1_moe_grouped_prepared_static(ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(),
                                              x.data_ptr(), tokens, stream)
    assert rc == -2 and b'static buffer serves' in lib.sub1_last_error()
    assert lib.sub1_moe_grouped_prepared_static(ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(),
                                                x.data_ptr(), 0, stream) == 0


def test_static_scratch_allocates_nothing_and_serves_stacks_of_different_widths(oracle):
    """Across calls of the entry point neither the device's free memory nor
    torch's pools move, and two stacks of different d_ff take turns on the one
    array: the wide one's h (many tokens) lies where a narrower stack's larger
    launch would keep control words if the array were laid out per call, which
    is why its split is fixed."""
    from qmoe_amd import _lib, sub1
    assert torch.cuda.is_available() and sub1.DEC
    lib = _lib.load()
    _lib.check(lib.sub1_init())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    wide, wi_w, wo_w = small_stack(oracle, 2, 256, 3072, 0.9, seed=1900)
    slim, wi_s, wo_s = small_stack(oracle, 3, 3072, 256, 0.9, seed=1950)
    prep_w, prep_s = wide.prepare(), slim.prepare()

    def run(prep, wi, wo, d_model, tokens, seed):
        experts = len(wi)
        route = [(7 * i + 1) % experts for i in range(tokens)]
        xs = np.stack([so.synthetic_activation(d_model, seed + i) for i in range(tokens)])
        x = bf16_dev(xs)
        te = torch.tensor(route, dtype=torch.int32, device='cuda')
        got = torch.full_like(x, 3.0)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        pools0 = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
        _lib.check(lib.sub1_moe_grouped_prepared_static(
            ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(), got.data_ptr(), tokens, stream))
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == pools0
        got = bits_host(got)
        for i in sorted({0, tokens // 2, tokens - 1}):
            ref, _ = oracle.expert_ffn(wi[route[i]], wo[route[i]], xs[i], order=2)
            assert np.array_equal(got[i], ref), (d_model, tokens, i)

    run(prep_w, wi_w, wo_w, 256, 1, 2000)       # warm-up: kernels loaded, attributes set
    run(prep_s, wi_s, wo_s, 3072, 1, 2001)
    run(prep_w, wi_w, wo_w, 256, 34, 2010)      # h of 34 x 3072 values at the array's end
    run(prep_s, wi_s, wo_s, 3072, 200, 2020)    # 200 tokens' words, far into the array
    run(prep_w, wi_w, wo_w, 256, 34, 2030)
    run(prep_s, wi_s, wo_s, 3072, 3, 2040)
    _lib.check_faults()


def test_static_scratch_launch_replays_from_a_graph(oracle):
    """The launch records kernel nodes only (no allocation, no memset node):
    captured once, it replays with the eager result every time, with eager
    launches on the same array and synchronisations between the replays."""
    from qmoe_amd import _lib, sub1
    assert torch.cuda.is_available() and sub1.DEC
    lib = _lib.load()
    _lib.check(lib.sub1_init())
    experts, d_model, d_ff = 4, 768, 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=2100)
    prep = stack.prepare()
    for tokens in (2, 9):
        route = [(3 * i + 1) % experts for i in range(tokens)]
        te = torch.tensor(route, dtype=torch.int32, device='cuda')
        x = bf16_dev(np.stack([so.synthetic_activation(d_model, 2200 + i) for i in range(tokens)]))
        y = torch.empty_like(x)

        def launch(out):
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            _lib.check(lib.sub1_moe_grouped_prepared_static(
                ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(), out.data_ptr(), tokens, stream))

        launch(y)                                # eager first: kernels loaded, attributes set
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            launch(y)
        for rep in range(3):
            xs = np.stack([so.synthetic_activation(d_model, 2300 + 10 * rep + i) for i in range(tokens)])
            x.copy_(bf16_dev(xs))
            y.zero_()
            graph.replay()
            torch.cuda.synchronize()
            got = bits_host(y)
            eager = torch.empty_like(x)
            launch(eager)                        # eager work on the same array between replays
            torch.cuda.synchronize()
            assert np.array_equal(got, bits_host(eager)), (tokens, rep)
            ref, _ = oracle.expert_ffn(wi[route[0]], wo[route[0]], xs[0], order=2)
            assert np.array_equal(got[0], ref)
    _lib.check_faults()
