"""What a launch cannot return as a status: a wait between workgroups that
gives up at its time limit, and a dec buffer that changed under the table
cached for its address.  Both are forced from the host (a tiny time limit and
a count no workgroup will ever reach; an overwritten tensor), every kernel
exits normally, and the sticky flags bring the condition to forward() and
check_faults()."""
import numpy as np
import pytest
import torch

from oracle import sub1_oracle as so
from test_gpu_parity import bf16_dev, bits_host, small_stack

pytestmark = pytest.mark.gpu


@pytest.fixture()
def lib():
    from qmoe_amd import _lib, sub1
    assert torch.cuda.is_available() and sub1.DEC
    handle = _lib.load()
    _lib.check(handle.sub1_init())
    _lib.clear_faults()
    yield handle
    # whatever the test did: normal waits, normal limit, flags down
    handle.sub1_test_overstate_wait(0)
    handle.sub1_set_wait_limit_us(250000)
    torch.cuda.synchronize()
    _lib.clear_faults()


@pytest.mark.parametrize('form', ['prepared', 'packed', 'tagged', 'tagged_split'])
def test_a_wait_that_gives_up_is_reported(lib, oracle, form):
    from qmoe_amd import _lib, sub1_hip
    # (rows of wo as long as d_ff = 8192 makes them: wo gets workgroups of its own)
    experts, d_model, d_ff = 3, 768, 8192 if form == 'tagged_split' else 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=900)
    runner = stack if form == 'packed' else stack.prepare()
    # two tokens: the launch whose workgroups wait for tagged values instead of a count
    route = [2, 1] if form.startswith('tagged') else [0, 1, 2, 1, 0, 2]
    xs = np.stack([so.synthetic_activation(d_model, 950 + i) for i in range(len(route))])
    x, te = bf16_dev(xs), torch.tensor(route, dtype=torch.int32, device='cuda')
    order = 1 if form == 'packed' else 2
    want = np.stack([oracle.expert_ffn(wi[e], wo[e], xs[i], order=order)[0]
                     for i, e in enumerate(route)])
    assert np.array_equal(bits_host(runner.forward(x, te)), want)
    assert runner.launch_faults(len(route)) == (0, 0)
    sub1_hip.check_faults()
    # a kernel whose workgroups wait for each other (whole tokens per workgroup do not)
    if form.startswith('tagged'):
        assert lib.sub1_last_kernel().decode() == 'moe_prepared_' + form + '_kernel'
    else:
        assert lib.sub1_last_kernel().decode() in ('moe_prepared_shared_kernel', 'moe_prepared_kernel',
                                                   'moe_prepared_small_kernel', 'moe_kernel<256>')

    # every wait of the next launch expects one workgroup more than exists and
    # may last 300 us: each gives up, the kernel still runs to its end
    _lib.check(lib.sub1_set_wait_limit_us(300))
    _lib.check(lib.sub1_test_overstate_wait(1))
    runner.forward(x, te)
    torch.cuda.synchronize()
    gave_up, bad_ids = runner.launch_faults(len(route))
    assert gave_up > 0 and bad_ids == 0
    flags = (np.ctypeslib.ctypes.c_int32 * 2)()
    _lib.check(lib.sub1_fault_flags(flags))
    assert flags[0] == 1 and flags[1] == 0
    with pytest.raises(sub1_hip.Sub1Fault, match='time limit'):
        sub1_hip.check_faults()
    with pytest.raises(sub1_hip.Sub1Fault):          # sticky: the next forward refuses
        runner.forward(x, te)

    # back to normal: flags cleared, the same launch is right again
    _lib.check(lib.sub1_test_overstate_wait(0))
    _lib.check(lib.sub1_set_wait_limit_us(250000))
    sub1_hip.clear_faults()
    assert np.array_equal(bits_host(runner.forward(x, te)), want)
    torch.cuda.synchronize()
    assert runner.launch_faults(len(route)) == (0, 0)
    sub1_hip.check_faults()


def test_wait_limit_arguments(lib):
    from qmoe_amd import _lib
    assert lib.sub1_set_wait_limit_us(0) != 0
    assert lib.sub1_set_wait_limit_us(10 ** 9) != 0
    assert lib.sub1_test_overstate_wait(-1) != 0
    _lib.check(lib.sub1_set_wait_limit_us(250000))


def test_an_address_that_holds_another_dictionary(lib, oracle):
    """The grouped launch on the packed layout caches its compact table by the
    address of dec.  The same tensor overwritten with another table: the next
    launch still multiplies by the old one but says so; after clear_faults()
    the table is derived afresh.  The single product reads dec itself and
    follows the new contents at once."""
    from qmoe_amd import _lib, sub1, sub1_hip
    d_model, d_ff = 130, 96
    ti, mi = so.synthetic_ternary(d_ff, d_model, 0.6, 77)
    to, mo = so.synthetic_ternary(d_model, d_ff, 0.6, 79)
    wi, wo = oracle.encode(ti) + (mi,), oracle.encode(to) + (mo,)
    xv = so.synthetic_activation(d_model, 78)
    dev = lambda l: (torch.from_numpy(l[0].view(np.int16)).cuda(),
                     torch.from_numpy(l[1]).cuda(), bf16_dev(l[2]))
    mine = sub1.DEC[0].clone()
    stack = sub1_hip.ExpertStack.from_layers(mine, [dev(wi)], [dev(wo)])
    x = bf16_dev(xv[None, :])
    te = torch.zeros(1, dtype=torch.int32, device='cuda')
    want, _ = oracle.expert_ffn(wi, wo, xv, order=1)

    def layer():
        y = stack.forward(x, te)
        torch.cuda.synchronize()
        return bits_host(y)[0]

    def product():
        y = torch.zeros(d_ff, dtype=torch.bfloat16, device='cuda')
        dwi = dev(wi)
        sub1_hip.sub1matvec(mine, dwi[0], dwi[1], dwi[2], x[0], y)
        torch.cuda.synchronize()
        return bits_host(y)

    assert np.array_equal(layer(), want)
    assert np.array_equal(product(), oracle.matvec_wave(wi[0], wi[1], mi, xv))
    sub1_hip.check_faults()
    # every entry becomes "one pair of zeros": all products are zero under this table
    mine.fill_(1)
    assert not product().any()                       # the single product reads dec itself
    assert np.array_equal(layer(), want)             # the stale table, and the flag
    with pytest.raises(sub1_hip.Sub1Fault, match='dec'):
        sub1_hip.check_faults()
    sub1_hip.clear_faults()                          # drops the cached tables as well
    assert not layer().any()
    sub1_hip.check_faults()
    # and the explicit way: tell the library before the address changes hands
    _lib.check(lib.sub1_unregister_dec(mine.data_ptr()))
    mine.copy_(sub1.DEC[0])
    assert np.array_equal(layer(), want)
    sub1_hip.check_faults()
    _lib.check(lib.sub1_unregister_dec(mine.data_ptr()))


def test_launches_of_one_stack_on_two_streams(lib, oracle):
    """One stack, two streams: each stream has its own workspace, so the
    launches may overlap; both give the oracle's bits."""
    experts, d_model, d_ff = 4, 768, 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=1200)
    prep = stack.prepare()
    routes = ([0, 1, 2, 3, 1, 0], [3, 3, 0])
    xs = [np.stack([so.synthetic_activation(d_model, 1300 + 10 * k + i) for i in range(len(r))])
          for k, r in enumerate(routes)]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    outs = [[], []]
    for rep in range(5):
        for k, s in enumerate(streams):
            with torch.cuda.stream(s):
                x = bf16_dev(xs[k])
                te = torch.tensor(routes[k], dtype=torch.int32, device='cuda')
                outs[k].append(prep.forward(x, te))
    torch.cuda.synchronize()
    assert len(prep._ws) >= 2
    for k, r in enumerate(routes):
        want = np.stack([oracle.expert_ffn(wi[e], wo[e], xs[k][i], order=2)[0]
                         for i, e in enumerate(r)])
        for y in outs[k]:
            assert np.array_equal(bits_host(y), want)


@pytest.mark.parametrize('static', [False, True])
def test_control_words_left_behind_by_a_wait_fault_are_cleared(lib, oracle, static):
    """A wait that gives up can leave a token's control word at another value
    than zero (a workgroup that reports after the waiters have gone), which no
    later launch would notice.  Here the host writes such a word after a forced
    give-up; clear_faults() must make the next launch from the same stack (and
    from the static scratch) right again."""
    import ctypes
    from qmoe_amd import _lib, sub1_hip
    experts, d_model, d_ff = 3, 768, 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=960)
    prep = stack.prepare()
    route = [0, 1, 2, 1, 0, 2]
    xs = np.stack([so.synthetic_activation(d_model, 970 + i) for i in range(len(route))])
    x, te = bf16_dev(xs), torch.tensor(route, dtype=torch.int32, device='cuda')
    want = np.stack([oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)[0] for i, e in enumerate(route)])
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def forward():
        if not static:
            return prep.forward(x, te)
        y = torch.empty_like(x)
        _lib.check(lib.sub1_moe_grouped_prepared_static(
            ctypes.byref(prep._c), te.data_ptr(), x.data_ptr(), y.data_ptr(), len(route), stream))
        return y

    assert np.array_equal(bits_host(forward()), want)
    assert lib.sub1_last_kernel().decode() == 'moe_prepared_shared_kernel'
    _lib.check(lib.sub1_set_wait_limit_us(300))
    _lib.check(lib.sub1_test_overstate_wait(1))
    forward()
    torch.cuda.synchronize()
    _lib.check(lib.sub1_test_overstate_wait(0))
    _lib.check(lib.sub1_set_wait_limit_us(250000))
    with pytest.raises(sub1_hip.Sub1Fault):
        sub1_hip.check_faults()
    # what a late writer leaves behind: one report and one wait on token 1's word
    epoch = lib.sub1_fault_epoch()
    words = torch.tensor([0x10001], dtype=torch.int32, device='cuda')
    at = _lib.load().sub1_moe_workspace_bytes(0, 0) + 64          # head, then 64 bytes per token
    if static:
        base = ctypes.c_void_p()
        _lib.check(lib.sub1_static_scratch_pointer(ctypes.byref(base)))
        hip = ctypes.CDLL('libamdhip64.so')
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        assert hip.hipMemcpy(base.value + at, words.data_ptr(), 4, 3) == 0     # device to device
    else:
        ws = prep.workspace(len(route))
        ws[at:at + 4].copy_(words.view(torch.uint8))
    torch.cuda.synchronize()
    sub1_hip.clear_faults()
    assert lib.sub1_fault_epoch() == epoch + 1
    assert np.array_equal(bits_host(forward()), want)
    torch.cuda.synchronize()
    sub1_hip.check_faults()
