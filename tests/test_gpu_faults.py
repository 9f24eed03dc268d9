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


@pytest.mark.parametrize('form', ['prepared', 'packed'])
def test_a_wait_that_gives_up_is_reported(lib, oracle, form):
    from qmoe_amd import _lib, sub1_hip
    experts, d_model, d_ff = 3, 768, 3072
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.9, seed=900)
    runner = stack.prepare() if form == 'prepared' else stack
    route = [0, 1, 2, 1, 0, 2]
    xs = np.stack([so.synthetic_activation(d_model, 950 + i) for i in range(len(route))])
    x, te = bf16_dev(xs), torch.tensor(route, dtype=torch.int32, device='cuda')
    order = 2 if form == 'prepared' else 1
    want = np.stack([oracle.expert_ffn(wi[e], wo[e], xs[i], order=order)[0]
                     for i, e in enumerate(route)])
    assert np.array_equal(bits_host(runner.forward(x, te)), want)
    assert runner.launch_faults(len(route)) == (0, 0)
    sub1_hip.check_faults()
    # a kernel whose workgroups wait for each other (whole tokens per workgroup do not)
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
    """sub1matvec caches its compact table by the address of dec.  The same
    tensor overwritten with another table: the next launch still multiplies by
    the old one but says so; after clear_faults() the table is derived afresh."""
    from qmoe_amd import _lib, sub1, sub1_hip
    height, width = 96, 130
    t, mm = so.synthetic_ternary(height, width, 0.6, 77)
    codes, row_off = oracle.encode(t)
    xv = so.synthetic_activation(width, 78)
    w_comp = torch.from_numpy(codes.view(np.int16)).cuda()
    ro, mmd, x = torch.from_numpy(row_off).cuda(), bf16_dev(mm), bf16_dev(xv)
    mine = sub1.DEC[0].clone()
    want = oracle.matvec_seq(codes, row_off, mm, xv)

    def product():
        y = torch.zeros(height, dtype=torch.bfloat16, device='cuda')
        sub1_hip.sub1matvec(mine, w_comp, ro, mmd, x, y)
        torch.cuda.synchronize()
        return bits_host(y)

    assert np.array_equal(product(), want)
    sub1_hip.check_faults()
    # every entry becomes "one pair of zeros": all products are zero under this table
    mine.fill_(1)
    assert np.array_equal(product(), want)           # the stale table, and the flag
    with pytest.raises(sub1_hip.Sub1Fault, match='dec'):
        sub1_hip.check_faults()
    sub1_hip.clear_faults()                          # drops the cached tables as well
    assert not product().any()
    sub1_hip.check_faults()
    # and the explicit way: tell the library before the address changes hands
    _lib.check(lib.sub1_unregister_dec(mine.data_ptr()))
    mine.copy_(sub1.DEC[0])
    assert np.array_equal(product(), want)
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
