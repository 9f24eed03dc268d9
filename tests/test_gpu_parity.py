"""GPU parity tests: the HIP library, called through its C ABI (via the ctypes
binding), against the CPU oracle on the same seeded inputs.

Bars:
  * decode, pack: bit-exact against the oracle (integer/byte work);
  * products: the output must equal, bit for bit, the oracle's result in the
    order the kernel adds in (wavefront-per-row order for the single product
    on the packed layout, per-symbol stream order for the grouped launch on
    it, prepared-stream order for the prepared kernels), must lie within
        2^-8 |exact| + 64 * 2^-24 * sum|w x|
    of the double-precision product, and must agree with the reference kernel's
    lane-order arithmetic to 1e-2 relative (normwise), the tolerance the task
    states for bf16 outputs with fp32 accumulation.
"""
import numpy as np
import pytest
import torch

from oracle import sub1_oracle as so

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2          # stated tolerance for outputs

SWITCH_SHAPES = [(3072, 768, 0.90), (768, 3072, 0.90), (4096, 1024, 0.88),
                 (1024, 4096, 0.88), (6144, 2080, 0.90), (2080, 6144, 0.90)]
ODD_SHAPES = [(77, 333, 0.7), (5, 1, 0.5), (9, 2, 0.5), (33, 29, 0.3), (64, 56, 0.0),
              (130, 15, 0.9), (1, 4000, 0.95), (300, 12288, 0.99), (2, 13000, 0.97)]


@pytest.fixture(scope='module')
def gpu():
    from qmoe_amd import sub1, sub1_hip
    assert torch.cuda.is_available(), 'these tests need the GPU'
    assert sub1.DEC, 'device tables missing'
    return sub1, sub1_hip


def bf16_dev(bits):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)


def bits_host(t):
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def dev_case(oracle, height, width, p0, seed):
    t, mm = so.synthetic_ternary(height, width, p0, seed)
    codes, row_off = oracle.encode(t)
    x = so.synthetic_activation(width, seed + 1000)
    d = dict(t=t, mm=mm, codes=codes, row_off=row_off, x=x,
             w_comp=torch.from_numpy(codes.view(np.int16)).cuda(),
             row_off_d=torch.from_numpy(row_off).cuda(), mm_d=bf16_dev(mm), x_d=bf16_dev(x))
    return d


def close(a, b):
    """Two bf16 results of the same product, summed in different orders."""
    a, b = a.float().double(), b.float().double()
    return bool(torch.linalg.norm(a - b) <= REL_TOL * torch.linalg.norm(b))


def check_product(oracle, c, y_bits, prepared=False):
    exact, sum_abs = oracle.matvec_f64(c['t'].astype(np.uint8), c['mm'], c['x'])
    y = so.bf16_bits_to_f32(y_bits).astype(np.float64)
    bound = 2.0 ** -8 * np.abs(exact) + 64 * 2.0 ** -24 * sum_abs + 1e-30
    assert np.all(np.abs(y - exact) <= bound)
    lanes = so.bf16_bits_to_f32(oracle.matvec_lanes(c['codes'], c['row_off'], c['mm'], c['x']))
    denom = max(np.linalg.norm(lanes), 1e-30)
    assert np.linalg.norm(y - lanes) / denom <= REL_TOL
    fn = oracle.matvec_gap if prepared else oracle.matvec_wave
    assert np.array_equal(y_bits, fn(c['codes'], c['row_off'], c['mm'], c['x']))


def test_device_tables_equal_oracle(gpu, oracle):
    sub1, _ = gpu
    dec, trie = oracle.tables()
    assert np.array_equal(sub1.DEC[0].cpu().numpy(), dec)
    assert np.array_equal(sub1.TRIE.cpu().numpy(), trie)


@pytest.mark.parametrize('height,width,p0', SWITCH_SHAPES + ODD_SHAPES)
def test_decode_bit_exact(gpu, oracle, height, width, p0):
    sub1, op = gpu
    c = dev_case(oracle, height, width, p0, seed=height + width)
    tern, w, bad = op.sub1decode(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    assert bad == 0
    assert np.array_equal(tern.cpu().numpy(), c['t'].astype(np.uint8))
    assert np.array_equal(bits_host(w), oracle.dequant(c['t'].astype(np.uint8), c['mm']))


def test_decode_counts_bad_rows(gpu, oracle):
    sub1, op = gpu
    c = dev_case(oracle, 8, 64, 0.9, seed=1)
    ro = c['row_off'].copy()
    ro[3] -= 1                                   # row 2 loses a code, row 3 gains one
    _, _, bad = op.sub1decode(sub1.DEC[0], c['w_comp'], torch.from_numpy(ro).cuda(),
                              c['mm_d'], 64, want_w=False)
    assert bad == 2


@pytest.mark.parametrize('height,width,p0', SWITCH_SHAPES + ODD_SHAPES)
def test_pack_bit_exact(gpu, oracle, height, width, p0):
    sub1, op = gpu
    t, _ = so.synthetic_ternary(height, width, p0, seed=3 * height + width)
    codes, row_off = oracle.encode(t)
    w_tern = torch.from_numpy(t).cuda()
    ro = torch.full((height + 1,), -7, dtype=torch.int32, device='cuda')
    w_comp = op.sub1pack(sub1.TRIE, w_tern, ro)
    assert w_comp.dtype == torch.int16
    assert np.array_equal(ro.cpu().numpy(), row_off)
    assert np.array_equal(w_comp.cpu().numpy().view(np.uint16), codes)


@pytest.mark.parametrize('height,width,p0', SWITCH_SHAPES + ODD_SHAPES)
def test_matvec_against_oracle(gpu, oracle, height, width, p0):
    sub1, op = gpu
    c = dev_case(oracle, height, width, p0, seed=7 * height + width)
    y = torch.zeros(height, dtype=torch.bfloat16, device='cuda')
    op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], c['x_d'], y)
    check_product(oracle, c, bits_host(y))


def test_matvec_accumulates_into_y(gpu, oracle):
    sub1, op = gpu
    c = dev_case(oracle, 200, 512, 0.9, seed=5)
    pre = so.f32_to_bf16_bits(np.random.default_rng(0).standard_normal(200).astype(np.float32))
    y = bf16_dev(pre).clone()
    op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], c['x_d'], y)
    want = oracle.matvec_wave(c['codes'], c['row_off'], c['mm'], c['x'], y=pre)
    assert np.array_equal(bits_host(y), want)
    # twice more: the reference's benchmark loop keeps adding onto y (test.py:175)
    op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], c['x_d'], y)
    want = oracle.matvec_wave(c['codes'], c['row_off'], c['mm'], c['x'], y=want)
    assert np.array_equal(bits_host(y), want)


def test_matvec_closed_forms(gpu, oracle):
    sub1, op = gpu
    c = dev_case(oracle, 96, 300, 0.6, seed=9)
    w = so.bf16_bits_to_f32(oracle.dequant(c['t'].astype(np.uint8), c['mm']))
    for k in (0, 1, 27, 28, 150, 299):
        x = torch.zeros(300, dtype=torch.bfloat16, device='cuda')
        x[k] = 1.0
        y = torch.zeros(96, dtype=torch.bfloat16, device='cuda')
        op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], x, y)
        assert np.array_equal(y.float().cpu().numpy(), w[:, k])
    x = torch.ones(300, dtype=torch.bfloat16, device='cuda')
    y = torch.zeros(96, dtype=torch.bfloat16, device='cuda')
    op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], x, y)
    f = so.bf16_bits_to_f32(c['mm'])
    n1, n2 = (c['t'] == 1).sum(1), (c['t'] == 2).sum(1)
    want = so.f32_to_bf16_bits((f[0::2] * n1 + f[1::2] * n2).astype(np.float32))
    assert np.array_equal(bits_host(y), want)


def test_matvec_on_unaligned_views(gpu, oracle):
    """x[i] / y[i] row views and a code stream that starts at an odd element,
    as the callers at reference sub1.py:141 and an expert stack produce."""
    sub1, op = gpu
    c = dev_case(oracle, 130, 333, 0.8, seed=12)
    pad = torch.zeros(3, dtype=torch.int16, device='cuda')
    stream = torch.cat((pad, c['w_comp']))[3:]
    assert stream.data_ptr() % 4 == 2
    xs = torch.zeros((3, 333), dtype=torch.bfloat16, device='cuda')
    xs[1] = c['x_d']
    ys = torch.zeros((3, 130), dtype=torch.bfloat16, device='cuda')
    op.sub1matvec(sub1.DEC[0], stream, c['row_off_d'], c['mm_d'], xs[1], ys[1])
    check_product(oracle, c, bits_host(ys[1]))
    assert not ys[0].any() and not ys[2].any()


def test_matvec_rejects_bad_tensors(gpu, oracle):
    sub1, op = gpu
    c = dev_case(oracle, 16, 64, 0.9, seed=2)
    y = torch.zeros(16, dtype=torch.bfloat16, device='cuda')
    with pytest.raises(TypeError):
        op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], c['x_d'].float(), y)
    with pytest.raises(ValueError):
        op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], c['x_d'].cpu(), y)
    with pytest.raises(ValueError):
        op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'][:-1], c['mm_d'], c['x_d'], y)
    with pytest.raises(ValueError):
        op.sub1matvec(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'][:-2], c['x_d'], y)
    with pytest.raises(TypeError):
        op.sub1matvec(sub1.DEC[0], c['w_comp'].int(), c['row_off_d'], c['mm_d'], c['x_d'], y)


def test_matvec_tokens(gpu, oracle):
    sub1, op = gpu
    c = dev_case(oracle, 300, 768, 0.9, seed=21)
    xs = np.stack([so.synthetic_activation(768, 50 + i) for i in range(5)])
    y = torch.zeros((5, 300), dtype=torch.bfloat16, device='cuda')
    op.sub1matvec_tokens(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], bf16_dev(xs), y)
    for i in range(5):
        want = oracle.matvec_wave(c['codes'], c['row_off'], c['mm'], xs[i])
        assert np.array_equal(bits_host(y[i]), want)


@pytest.mark.parametrize('height,width,p0', [(3072, 768, 0.9), (768, 3072, 0.9), (96, 130, 0.4)])
def test_sub1linear_make_and_forward(gpu, oracle, height, width, p0):
    """The reference's own smoke check (test.py:180-189): dense product, kernel
    product and make(w) round trip must agree."""
    sub1, op = gpu
    t, mm = so.synthetic_ternary(height, width, p0, seed=31)
    assert (t == 1).any(1).all() and (t == 2).any(1).all()   # make() needs both signs per row
    w_bits = oracle.dequant(t.astype(np.uint8), mm)
    w = bf16_dev(w_bits)
    lin = sub1.Sub1Linear.make(w)
    codes, row_off = oracle.encode(t)
    assert np.array_equal(lin.row_off.cpu().numpy(), row_off)
    assert np.array_equal(lin.w_comp.cpu().numpy().view(np.uint16), codes)
    assert np.array_equal(bits_host(lin.ter_minmax), mm)
    x = torch.randn((3, width), generator=torch.Generator().manual_seed(1)).bfloat16().cuda()
    y = lin(x)
    assert y.shape == (3, height) and y.dtype == torch.bfloat16
    ref = x.float() @ w.float().t()                       # plain fp32 torch reference
    err = (y.float() - ref).norm() / ref.norm()
    assert err <= REL_TOL
    assert lin(x[:0]).shape == (0, height)


def small_stack(oracle, experts, d_model, d_ff, p0, seed):
    from qmoe_amd import sub1, sub1_hip
    wi, wo = [], []
    for e in range(experts):
        ti, mi = so.synthetic_ternary(d_ff, d_model, p0, seed + 2 * e)
        to, mo = so.synthetic_ternary(d_model, d_ff, p0, seed + 2 * e + 1)
        wi.append(oracle.encode(ti) + (mi,))
        wo.append(oracle.encode(to) + (mo,))
    dev = lambda l: (torch.from_numpy(l[0].view(np.int16)).cuda(),
                     torch.from_numpy(l[1]).cuda(), bf16_dev(l[2]))
    stack = sub1_hip.ExpertStack.from_layers(sub1.DEC[0], [dev(l) for l in wi],
                                             [dev(l) for l in wo])
    return stack, wi, wo


@pytest.mark.parametrize('experts,d_model,d_ff,p0', [(6, 96, 200, 0.8), (4, 768, 3072, 0.9),
                                                     (3, 333, 77, 0.7)])
def test_grouped_launch_against_oracle(gpu, oracle, experts, d_model, d_ff, p0):
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, p0, seed=100)
    # skewed routing: expert 0 gets several tokens, the last expert none, one
    # token is dropped (-1) and one names an expert that does not exist
    route = [0, 1, 0, -1, 2 % experts, 0, experts + 5, 1, 0]
    xs = np.stack([so.synthetic_activation(d_model, 200 + i) for i in range(len(route))])
    x = bf16_dev(xs)
    y = stack.forward(x, torch.tensor(route, dtype=torch.int32, device='cuda'))
    got = bits_host(y)
    assert stack.launch_faults(len(route)) == (0, 1)
    for i, e in enumerate(route):
        if e < 0 or e >= experts:
            assert np.array_equal(got[i], xs[i])
        else:
            want, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=1)
            assert np.array_equal(got[i], want), (i, e)
            lanes, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=0)
            a, b = so.bf16_bits_to_f32(got[i]), so.bf16_bits_to_f32(lanes)
            assert np.linalg.norm(a - b) <= REL_TOL * np.linalg.norm(b)
    # a second launch reuses the workspace
    y2 = stack.forward(x, torch.tensor(route, dtype=torch.int32, device='cuda'))
    assert torch.equal(y, y2)


@pytest.mark.parametrize('experts,d_model,d_ff,p0', [(4, 768, 3072, 0.9), (3, 333, 77, 0.7),
                                                     (2, 2080, 6144, 0.9)])
def test_grouped_launch_in_its_sweep_form_against_oracle(gpu, oracle, experts, d_model, d_ff, p0):
    """With at least a token per compute unit the packed-layout launch runs one
    workgroup of 16 wavefronts per compute unit, whole projections as tiles (a
    thread takes rows in turn) and the head of the table from LDS: the same
    sums in the same order, so sampled tokens equal the oracle to the bit,
    dropped and out-of-range tokens keep their input."""
    from qmoe_amd import _lib
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, p0, seed=150)
    tokens = 300
    route = [(5 * i + 1) % experts for i in range(tokens)]
    route[7], route[123], route[299] = -1, experts + 2, -1
    xs = np.stack([so.synthetic_activation(d_model, 250 + i) for i in range(tokens)])
    x = bf16_dev(xs)
    te = torch.tensor(route, dtype=torch.int32, device='cuda')
    y = stack.forward(x, te)
    assert _lib.load().sub1_last_kernel() == b'moe_kernel<1024>'
    got = bits_host(y)
    assert stack.launch_faults(tokens) == (0, 1)
    for i in (0, 1, 7, 64, 123, 150, 298, 299):
        e = route[i]
        if e < 0 or e >= experts:
            assert np.array_equal(got[i], xs[i]), i
        else:
            want, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=1)
            assert np.array_equal(got[i], want), (i, e)
    # the same tokens a few at a time go through the other form of the launch: the same bits
    few = stack.forward(x[:9].contiguous(), te[:9].contiguous())
    assert _lib.load().sub1_last_kernel() == b'moe_kernel<256>'
    assert torch.equal(few, y[:9])
    assert torch.equal(stack.forward(x, te), y)


def test_grouped_launch_no_tokens_and_all_dropped(gpu, oracle):
    stack, _, _ = small_stack(oracle, 2, 64, 128, 0.8, seed=300)
    x = torch.zeros((0, 64), dtype=torch.bfloat16, device='cuda')
    assert stack.forward(x, torch.zeros(0, dtype=torch.int32, device='cuda')).shape == (0, 64)
    x = torch.randn((4, 64), device='cuda').bfloat16()
    y = stack.forward(x, torch.full((4,), -1, dtype=torch.int32, device='cuda'))
    assert torch.equal(x, y)


@pytest.mark.parametrize('experts,d_model,d_ff,p0', [(6, 96, 200, 0.8), (4, 768, 3072, 0.9),
                                                     (3, 333, 77, 0.7), (2, 2080, 6144, 0.9),
                                                     (2, 1024, 4096, 0.88)])
def test_prepared_stack_against_oracle(gpu, oracle, experts, d_model, d_ff, p0):
    """The fast path: same bars as the grouped launch (bit-exact in its own
    order of additions), and within the tolerance of it."""
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, p0, seed=400)
    prep = stack.prepare()
    route = [0, 1, 0, -1, 2 % experts, 0, experts + 5, 1, 0, experts - 1]
    xs = np.stack([so.synthetic_activation(d_model, 500 + i) for i in range(len(route))])
    x = bf16_dev(xs)
    te = torch.tensor(route, dtype=torch.int32, device='cuda')
    y = prep.forward(x, te)
    got = bits_host(y)
    assert prep.launch_faults(len(route)) == (0, 1)
    for i, e in enumerate(route):
        if e < 0 or e >= experts:
            assert np.array_equal(got[i], xs[i])
        else:
            want, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)
            assert np.array_equal(got[i], want), (i, e)
            lanes, _ = oracle.expert_ffn(wi[e], wo[e], xs[i], order=0)
            a, b = so.bf16_bits_to_f32(got[i]), so.bf16_bits_to_f32(lanes)
            assert np.linalg.norm(a - b) <= REL_TOL * np.linalg.norm(b)
    assert close(y, stack.forward(x, te))
    assert torch.equal(y, prep.forward(x, te))          # workspace reuse
    # the prepared stream holds every weight of every matrix
    for e in range(experts):
        for proj, layer, width in ((0, wi[e], d_model), (1, wo[e], d_ff)):
            want = oracle.decode(layer[0], layer[1], width)
            assert np.array_equal(prep.decode(e, proj).cpu().numpy(), want), (e, proj)


def test_prepared_stack_tiny_and_huge_activations(gpu, oracle):
    """bf16 subnormals and values near the top of the range through the
    dot-product instruction the fast path adds with."""
    stack, wi, wo = small_stack(oracle, 2, 128, 192, 0.6, seed=600)
    prep = stack.prepare()
    rng = np.random.default_rng(5)
    scales = [1e-40, 1e-38, 1e-30, 1.0, 1e30]
    xs = np.stack([so.f32_to_bf16_bits((rng.standard_normal(128) * sc).astype(np.float32))
                   for sc in scales])
    te = torch.tensor([0, 1, 0, 1, 0], dtype=torch.int32, device='cuda')
    got = bits_host(prep.forward(bf16_dev(xs), te))
    ref = bits_host(stack.forward(bf16_dev(xs), te))
    for i in range(len(scales)):
        a, b = so.bf16_bits_to_f32(got[i]).astype(np.float64), so.bf16_bits_to_f32(ref[i]).astype(np.float64)
        assert np.all(np.isfinite(a))
        assert np.linalg.norm(a - b) <= REL_TOL * max(np.linalg.norm(b), 1e-37), scales[i]


def test_prepare_rejects_foreign_dictionary(gpu, oracle):
    from qmoe_amd._lib import Sub1Error
    from qmoe_amd import sub1, sub1_hip
    stack, _, _ = small_stack(oracle, 2, 64, 128, 0.8, seed=700)
    other = sub1.DEC[0].clone()
    other[5] += 16
    bad = sub1_hip.ExpertStack(other, stack.w_comp, stack.wi_code_base, stack.wo_code_base,
                               stack.wi_row_off, stack.wo_row_off, stack.wi_minmax,
                               stack.wo_minmax, 64, 128)
    with pytest.raises(Sub1Error):
        bad.prepare()


def test_prepare_rejects_rows_that_do_not_cover_the_width(gpu, oracle):
    """A row_off that cuts a row's codes short (or a width the codes were not
    made for) is refused when the stream is prepared, not decoded into garbage."""
    from qmoe_amd._lib import Sub1Error
    sub1, op = gpu
    c = dev_case(oracle, 96, 200, 0.8, seed=710)
    bad = c['row_off_d'].clone()
    bad[40] -= 1                                  # row 39 loses a code, row 40 gains it
    with pytest.raises(Sub1Error):
        op.PreparedMatrix(sub1.DEC[0], c['w_comp'], bad, c['mm_d'], 200)
    with pytest.raises(Sub1Error):
        op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], 204)
    op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], 200)


def test_large_stack_paths_agree_and_match_oracle(gpu, oracle):
    """128 Switch-base experts, one token each (the Switch-base-128 layer):
    many tiles on many compute units, so the hand-off of the intermediate
    activations between workgroups is exercised.  Both kernels must repeat
    their results, agree within the tolerance, and match the oracle on sampled
    tokens, each in its own order of additions."""
    from qmoe_amd import synthetic
    experts, d_model, d_ff = 128, 768, 3072
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.9, seed=99)
    prep = stack.prepare()
    x = synthetic.activations(experts, d_model, seed=100)
    route = torch.arange(experts, dtype=torch.int32, device='cuda')
    y_ref = stack.forward(x, route).clone()
    y_prep = prep.forward(x, route).clone()
    assert close(y_prep, y_ref)
    for _ in range(5):
        assert torch.equal(prep.forward(x, route), y_prep)
        assert torch.equal(stack.forward(x, route), y_ref)
    assert prep.launch_faults(experts) == (0, 0)
    xs = bits_host(x)
    for e in (0, 17, 63, 127):
        wi, wo = synthetic.expert_layers(stack, e)
        host = [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                for l in (wi, wo)]
        for got, order in ((y_ref, 1), (y_prep, 2)):
            want, _ = oracle.expert_ffn(host[0], host[1], xs[e], order=order)
            assert np.array_equal(bits_host(got[e]), want), (e, order)


def test_routed_batch_equals_per_token_products(gpu):
    """64 tokens routed top-1 by a softmax router over c-2048-shaped experts
    (skewed per-expert counts, experts with no token): the one-launch result
    must equal what the per-token calls of the reference's loop give
    (sub1.py:139-142 and 315-317: wi product, ReLU, wo product per token),
    to the bit for kernels that add in the same order."""
    from qmoe_amd import sub1, sub1_hip, synthetic
    experts, d_model, d_ff, tokens = 48, 2080, 6144, 64
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.9, seed=5)
    prep = stack.prepare()
    x = synthetic.activations(tokens, d_model, seed=6)
    route = synthetic.softmax_router(tokens, experts, seed=7)
    counts = torch.bincount(route.long(), minlength=experts)
    assert counts.max() >= 2 and (counts == 0).any()        # skewed, some experts idle
    y = prep.forward(x, route).clone()
    y_packed = stack.forward(x, route)
    assert close(y, y_packed)
    dec = sub1.DEC[0]
    for t in range(tokens):
        # the packed-layout kernels, called per token like the reference's loop
        wi, wo = synthetic.expert_layers(stack, int(route[t]))
        h = torch.zeros(d_ff, dtype=torch.bfloat16, device='cuda')
        sub1_hip.sub1matvec(dec, wi[0], wi[1], wi[2], x[t], h)
        h = torch.relu(h)
        out = torch.zeros(d_model, dtype=torch.bfloat16, device='cuda')
        sub1_hip.sub1matvec(dec, wo[0], wo[1], wo[2], h, out)
        # (the single product adds a row by lanes of a wavefront, the grouped
        # launch on the packed layout codeword by codeword: rounding apart)
        assert close(out, y_packed[t]), t
        # the prepared kernels, one token per launch
        one = prep.forward(x[t:t + 1].contiguous(), route[t:t + 1].contiguous())
        assert torch.equal(one[0], y[t]), t


def test_every_tiling_mode_gives_the_same_bits(gpu, oracle):
    """The prepared kernels tile differently with the batch size: a token
    with both its matrices per workgroup (many tokens), whole matrices or
    parts of a matrix (fewer), several wavefronts sharing one row slice from
    position checkpoints (a handful).
    The same token must come out identical in all of them, and equal to the
    oracle."""
    from qmoe_amd import synthetic
    experts, d_model, d_ff = 3, 2080, 6144
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.9, seed=11)
    prep = stack.prepare()
    x1 = synthetic.activations(1, d_model, seed=12)
    want = None
    for tokens in (1, 2, 5, 40, 300, 700):
        x = x1.repeat(tokens, 1).contiguous()
        route = torch.full((tokens,), 2, dtype=torch.int32, device='cuda')
        route[0] = 1
        y = prep.forward(x, route)
        assert prep.launch_faults(tokens) == (0, 0)
        if want is None:
            want = y[0].clone()
            wi, wo = synthetic.expert_layers(stack, 1)
            host = [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                    for l in (wi, wo)]
            ref, _ = oracle.expert_ffn(host[0], host[1], bits_host(x1[0]), order=2)
            assert np.array_equal(bits_host(want), ref)
        assert torch.equal(y[0], want), tokens
        if tokens > 1:
            assert torch.equal(y[1], y[tokens - 1])


def test_token_per_workgroup_tiles_with_dropped_tokens(gpu, oracle):
    """At least one token per compute unit: a workgroup then runs both
    projections of a token with the intermediate activations kept on chip.
    Dropped tokens pass through, out-of-range expert ids are counted, and the
    rest equals the small-batch result of the same tokens."""
    from qmoe_amd import synthetic
    experts, d_model, d_ff, tokens = 5, 1024, 4096, 520
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.88, seed=21)
    prep = stack.prepare()
    x = synthetic.activations(tokens, d_model, seed=22)
    route = (torch.arange(tokens, dtype=torch.int32, device='cuda') * 7) % experts
    route[3] = -1
    route[400] = -1
    route[77] = experts
    route[519] = experts + 100
    y = prep.forward(x, route)
    assert prep.launch_faults(tokens) == (0, 2)
    for t in (3, 400, 77, 519):
        assert torch.equal(y[t], x[t])
    keep = [0, 1, 2, 4, 5, 76, 78, 255, 256, 399, 401, 518]
    idx = torch.tensor(keep, device='cuda')
    small = prep.forward(x[idx].contiguous(), route[idx].contiguous())
    assert torch.equal(y[idx], small)
    assert close(y, stack.forward(x, route))


@pytest.mark.parametrize('d_model,d_ff,p0', [(2080, 6144, 0.9), (200, 330, 0.8), (64, 4096, 0.9)])
def test_tokens_shared_between_workgroups(gpu, oracle, d_model, d_ff, p0):
    """Fewer tokens than half the compute units (for large experts up to two
    thirds, in two rounds of workgroups): several workgroups share a
    token, each taking every n-th slice of both projections, the intermediate
    activations crossing memory once.  Shapes with fewer slices than
    workgroups per token (some get nothing to walk) and rows that do not fill
    the last slice; dropped tokens pass through, out-of-range expert ids are
    counted; every token equals its single-token launch to the bit and the
    oracle's sum in the stream's order."""
    from qmoe_amd import synthetic
    experts = 4
    stack = synthetic.build_stack(experts, d_model, d_ff, p0, seed=31)
    prep = stack.prepare()
    for tokens in (2, 3, 7, 30, 100, 128, 150):
        x = synthetic.activations(tokens, d_model, seed=32 + tokens)
        route = (torch.arange(tokens, dtype=torch.int32, device='cuda') * 3) % experts
        bad = 0
        if tokens >= 7:
            route[1] = -1
            route[5] = experts + 2
            bad = 1
        y = prep.forward(x, route)
        assert prep.launch_faults(tokens) == (0, bad)
        for t in range(tokens):
            if int(route[t]) < 0 or int(route[t]) >= experts:
                assert torch.equal(y[t], x[t]), (tokens, t)
        for t in sorted({0, min(2, tokens - 1), tokens // 2, tokens - 1}):
            one = prep.forward(x[t:t + 1].contiguous(), route[t:t + 1].contiguous())
            assert torch.equal(one[0], y[t]), (tokens, t)
        assert close(y, stack.forward(x, route))
    t = 2
    wi, wo = synthetic.expert_layers(stack, int(route[t]))
    host = [tuple(bits_host(v) if v.dtype != torch.int32 else v.cpu().numpy() for v in l)
            for l in (wi, wo)]
    ref, _ = oracle.expert_ffn(host[0], host[1], bits_host(x[t]), order=2)
    assert np.array_equal(bits_host(y[t]), ref)


def test_one_or_two_tokens_dropped_or_out_of_range(gpu):
    """Launches of one or two tokens hand h over by tag and count nothing per
    token; a dropped token or one whose expert does not exist still passes
    through, is counted, and leaves the other token's result and the next
    launches on the workspace as they were."""
    from qmoe_amd import _lib, synthetic
    experts, d_model, d_ff = 3, 512, 1536
    prep = synthetic.build_stack(experts, d_model, d_ff, 0.85, seed=61).prepare()
    x = synthetic.activations(2, d_model, seed=62)
    both = prep.forward(x, torch.tensor([1, 2], dtype=torch.int32, device='cuda')).clone()
    assert _lib.load().sub1_last_kernel() == b'moe_prepared_tagged_kernel'
    for route, bad in (([-1, 2], 0), ([1, experts], 1), ([-1, -7], 0), ([experts + 5, -1], 1),
                       ([1, 2], 0)):
        y = prep.forward(x, torch.tensor(route, dtype=torch.int32, device='cuda'))
        assert prep.launch_faults(2) == (0, bad), route
        for t, e in enumerate(route):
            assert torch.equal(y[t], both[t] if 0 <= e < experts else x[t]), (route, t)
    for e, bad in ((-1, 0), (experts, 1), (1, 0)):
        y = prep.forward(x[:1].contiguous(), torch.tensor([e], dtype=torch.int32, device='cuda'))
        assert prep.launch_faults(1) == (0, bad), e
        assert torch.equal(y[0], both[0] if e == 1 else x[0]), e


def test_one_and_two_tokens_on_random_shapes(gpu, oracle):
    """One token (wo in workgroups of its own, two to a slice) and two tokens
    (the same where wo's rows are long, every workgroup in both projections
    otherwise) through seeded random shapes, among them wo rows of one group
    of chunks and of more than sixteen, slices that are not full and a single
    row: every token equal to the oracle to the bit, dropped tokens passed
    through, and the launches after one another on one workspace."""
    from qmoe_amd import _lib
    rng = np.random.default_rng(77)
    shapes = [(1, 1), (64, 64), (65, 130), (96, 9000), (700, 40), (130, 4096), (2080, 6144)]
    shapes += [(int(rng.integers(1, 900)), int(rng.integers(1, 7000))) for _ in range(8)]
    kernels = set()
    for n, (d_model, d_ff) in enumerate(shapes):
        p0 = float(rng.choice([0.5, 0.9, 0.97]))
        stack, wi, wo = small_stack(oracle, 3, d_model, d_ff, p0, seed=7000 + n)
        prep = stack.prepare()
        xs = so.f32_to_bf16_bits(rng.standard_normal((2, d_model)).astype(np.float32))
        for route in ([2], [0, 1], [1], [-1, 2], [1, 1]):
            x = bf16_dev(xs[:len(route)])
            y = prep.forward(x, torch.tensor(route, dtype=torch.int32, device='cuda'))
            kernels.add(_lib.load().sub1_last_kernel())
            assert prep.launch_faults(len(route)) == (0, 0)
            got = bits_host(y)
            for i, e in enumerate(route):
                want = xs[i] if e < 0 else oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)[0]
                assert np.array_equal(got[i], want), (d_model, d_ff, p0, route, i)
    assert {b'moe_prepared_tagged_split_kernel', b'moe_prepared_tagged_kernel'} <= kernels, kernels


def test_one_workspace_serves_batches_in_any_order(gpu):
    """A workspace made for the largest batch then serves smaller and larger
    ones in any order: a small launch's h must not land on the words a larger
    launch counts with afterwards (h lies at the end of the workspace, the
    words at its head).  Both layouts, every launch against the same launch on
    a fresh workspace."""
    from qmoe_amd import synthetic
    experts, d_model, d_ff = 4, 200, 330
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.8, seed=41)
    prep = stack.prepare()
    sizes = (150, 1, 150, 7, 100, 2, 128, 60, 150)
    xs = {t: synthetic.activations(t, d_model, seed=42 + t) for t in set(sizes)}
    route = {t: (torch.arange(t, dtype=torch.int32, device='cuda') * 3 + 1) % experts for t in xs}
    for layer in (prep, stack):
        want = {}
        for t in xs:
            layer._ws.clear()
            want[t] = layer.forward(xs[t], route[t]).clone()
        layer._ws.clear()
        for t in sizes:
            got = layer.forward(xs[t], route[t])
            assert torch.equal(got, want[t]), (type(layer).__name__, t)
        assert len(layer._ws) == 1
        assert layer.launch_faults(max(sizes)) == (0, 0)


def test_shared_token_launches_on_several_streams(gpu):
    """Launches whose workgroups wait for each other (several per token) from
    three streams at once: together they ask for three times the compute
    units, so none has all its workgroups on the GPU at the start.  Every
    launch still completes without running into its wait limit, with the
    results of the same launches made one after the other."""
    from qmoe_amd import synthetic
    d_model, d_ff = synthetic.SHAPES['large']
    tokens = 128
    preps = [synthetic.build_stack(16, d_model, d_ff, 0.88, seed=81 + i).prepare() for i in range(3)]
    xs = [synthetic.activations(tokens, d_model, seed=85 + i) for i in range(3)]
    route = (torch.arange(tokens, dtype=torch.int32, device='cuda') * 5) % 16
    want = [p.forward(x, route).clone() for p, x in zip(preps, xs)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in preps]
    ys = [torch.empty_like(x) for x in xs]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    for rep in range(40):
        for p, x, y, s in zip(preps, xs, ys, streams):
            with torch.cuda.stream(s):
                p.forward(x, route, y)
    torch.cuda.synchronize()
    for p, y, ref in zip(preps, ys, want):
        assert p.launch_faults(tokens) == (0, 0)
        assert torch.equal(y, ref)


@pytest.mark.parametrize('d_model,d_ff', [(64, 12288), (12288, 64), (2, 2)])
def test_extreme_widths_in_every_batch_regime(gpu, oracle, d_model, d_ff):
    """The widest activations the fast layout takes and the narrowest, from one
    token to more tokens than compute units: every regime must give the same
    bits, equal to the oracle's, and agree with the packed-layout kernel."""
    stack, wi, wo = small_stack(oracle, 2, d_model, d_ff, 0.95, seed=800)
    prep = stack.prepare()
    xs = np.stack([so.synthetic_activation(d_model, 900 + i) for i in range(3)])
    want, _ = oracle.expert_ffn(wi[1], wo[1], xs[0], order=2)
    for tokens in (1, 7, 90, 300):
        x = bf16_dev(np.tile(xs, (tokens // 3 + 1, 1))[:tokens])
        route = torch.ones(tokens, dtype=torch.int32, device='cuda')
        route[1::2] = 0
        y = prep.forward(x, route)
        assert prep.launch_faults(tokens) == (0, 0)
        assert close(y, stack.forward(x, route)), tokens
        assert np.array_equal(bits_host(y[0]), want), tokens
        if tokens > 6:
            assert torch.equal(y[6], y[0])   # the same activations and expert again


@pytest.mark.parametrize('height,width,p0', SWITCH_SHAPES + [(77, 333, 0.7), (5, 1, 0.5),
                                                             (130, 15, 0.9), (300, 8192, 0.99),
                                                             (64, 56, 0.0), (33, 29, 0.3),
                                                             (1, 4000, 0.95), (200, 8192, 0.9995),
                                                             (40, 12288, 0.97)])
def test_prepared_matrix_product(gpu, oracle, height, width, p0):
    """The single-matrix fast path (what Sub1Linear.forward uses): y += W x for
    several tokens, bit-exact against the oracle, accumulating like sub1matvec."""
    sub1, op = gpu
    c = dev_case(oracle, height, width, p0, seed=11 * height + width)
    pm = op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    tokens = 3
    xs = np.stack([c['x']] + [so.synthetic_activation(width, 900 + i) for i in range(tokens - 1)])
    pre = so.f32_to_bf16_bits(np.random.default_rng(1).standard_normal((tokens, height)).astype(np.float32))
    y = bf16_dev(pre).clone()
    pm.matvec_tokens(bf16_dev(xs), y)
    got = bits_host(y)
    for i in range(tokens):
        want = oracle.matvec_gap(c['codes'], c['row_off'], c['mm'], xs[i], y=pre[i])
        assert np.array_equal(got[i], want), i
    y0 = torch.zeros((1, height), dtype=torch.bfloat16, device='cuda')
    pm.matvec_tokens(c['x_d'].reshape(1, -1), y0)
    check_product(oracle, c, bits_host(y0[0]), prepared=True)
    assert np.array_equal(pm.decode().cpu().numpy(), c['t'])


def test_sub1linear_fast_and_packed_paths_agree(gpu, oracle):
    sub1, op = gpu
    t, mm = so.synthetic_ternary(3072, 768, 0.9, seed=77)
    w = bf16_dev(oracle.dequant(t.astype(np.uint8), mm))
    lin = sub1.Sub1Linear.make(w)
    x = torch.randn((4, 768), generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    y_fast = lin(x)
    lin.fast = False
    y_packed = lin(x)
    assert close(y_fast, y_packed) and not torch.equal(y_fast, torch.zeros_like(y_fast))
    # replacing a buffer invalidates the prepared copy
    lin.fast = True
    lin.ter_minmax = (lin.ter_minmax.float() * 2).bfloat16()
    assert torch.equal(lin(x).float(), 2 * y_fast.float())


def test_sub1linear_prepared_copy_follows_the_buffers(gpu, oracle):
    """In-place writes and `.data` replacement (as a checkpoint loader does)
    must both be seen by the cached fast layout, also when the allocator could
    hand the old address to the new tensor."""
    sub1, op = gpu
    layers = []
    for seed in (81, 82):
        t, mm = so.synthetic_ternary(256, 128, 0.8, seed=seed)
        layers.append(sub1.Sub1Linear.make(bf16_dev(oracle.dequant(t.astype(np.uint8), mm))))
    a, b = layers
    x = torch.randn((3, 128), generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    ya, yb = a(x).clone(), b(x).clone()
    assert not torch.equal(ya, yb)
    # in place: a takes b's min/max (same shape), result changes accordingly
    saved = a.ter_minmax.clone()
    a.ter_minmax.copy_(b.ter_minmax)
    a.fast = False
    want = a(x).clone()
    a.fast = True
    assert torch.equal(a(x), want) and not torch.equal(want, ya)
    a.ter_minmax.copy_(saved)
    assert torch.equal(a(x), ya)
    # replacement after the old storage was dropped: freshly allocated tensors
    # of the same sizes, which the caching allocator would place where the old
    # ones were if nothing held them
    nb = {n: getattr(b, n).clone() for n in ('w_comp', 'row_off', 'ter_minmax')}
    for n in nb:
        getattr(a, n).data = torch.empty(0, dtype=nb[n].dtype, device='cuda')
    for n in nb:
        fresh = torch.empty_like(nb[n])
        fresh.copy_(nb[n])
        getattr(a, n).data = fresh
    assert torch.equal(a(x), yb)


def test_prepared_matrix_set_with_token_matrix(gpu, oracle):
    """Several matrices of one shape behind one launch: token t uses matrix
    token_matrix[t]; a token whose index names no matrix adds nothing."""
    sub1, op = gpu
    height, width, count = 130, 200, 3
    cases = [dev_case(oracle, height, width, 0.8, seed=950 + i) for i in range(count)]
    pm = op.PreparedMatrix(sub1.DEC[0], [c['w_comp'] for c in cases],
                           [c['row_off_d'] for c in cases], [c['mm_d'] for c in cases], width)
    which = [0, 2, 1, 1, -1, 0, 7, 2, 2, 0, 1]
    xs = np.stack([so.synthetic_activation(width, 970 + i) for i in range(len(which))])
    y0 = np.stack([so.synthetic_activation(height, 990 + i) for i in range(len(which))])
    y = bf16_dev(y0).clone()
    pm.matvec_tokens(bf16_dev(xs), y, torch.tensor(which, dtype=torch.int32, device='cuda'))
    got = bits_host(y)
    for t, m in enumerate(which):
        if m < 0 or m >= count:
            assert np.array_equal(got[t], y0[t])
        else:
            c = cases[m]
            want = oracle.matvec_gap(c['codes'], c['row_off'], c['mm'], xs[t], y=y0[t])
            assert np.array_equal(got[t], want), (t, m)
    with pytest.raises(ValueError):
        pm.matvec_tokens(bf16_dev(xs), y)            # several matrices need token_matrix


def test_prepared_stream_edge_rows(gpu, oracle):
    """Rows the gap stream treats specially: no non-zero at all (no entries, the
    slice still has one chunk), one non-zero in the last column after a gap of
    many steps over zeros, no zero at all (one entry per column), a row whose
    min equals its max (the packer codes every weight as symbol 2), and rows of
    very different lengths in one 64-row slice."""
    sub1, op = gpu
    height, width = 70, 1500
    t, mm = so.synthetic_ternary(height, width, 0.9, seed=4242)
    t[0, :] = 0
    t[1, :] = 0
    t[1, width - 1] = 2
    t[2, :] = 1
    t[3, :] = 2
    t[4, :] = 0
    t[4, 0] = 1
    t[5, :] = 0
    t[5, 59] = 2                     # a step of exactly 127
    t[6, :] = 0
    t[6, 60] = 1                     # 128: one step too long
    t[65:, :] = 0                    # the second slice holds only empty rows
    mm[2 * 3] = mm[2 * 3 + 1]        # row 3: min == max
    codes, row_off = oracle.encode(t)
    x = so.synthetic_activation(width, 77)
    w_comp = torch.from_numpy(codes.view(np.int16)).cuda()
    pm = op.PreparedMatrix(sub1.DEC[0], w_comp, torch.from_numpy(row_off).cuda(), bf16_dev(mm), width)
    assert np.array_equal(pm.decode().cpu().numpy(), t)
    for tokens in (1, 3):
        xs = np.stack([x] * tokens)
        y = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
        pm.matvec_tokens(bf16_dev(xs), y)
        want = oracle.matvec_gap(codes, row_off, mm, x)
        for i in range(tokens):
            assert np.array_equal(bits_host(y[i]), want)
    assert want[0] == 0 and want[70 - 1] == 0
    c = dict(t=t, mm=mm, codes=codes, row_off=row_off, x=x)
    check_product(oracle, c, want, prepared=True)


@pytest.mark.parametrize('height,width,p0,tokens', [(3072, 768, 0.9, 171), (768, 3072, 0.9, 513),
                                                    (77, 333, 0.7, 510), (130, 15, 0.9, 509),
                                                    (6144, 2080, 0.9, 86), (5, 1, 0.5, 515),
                                                    (200, 12288, 0.97, 511)])
def test_prepared_matrix_many_tokens(gpu, oracle, height, width, p0, tokens):
    """Enough tokens through one matrix that the launch walks the stream once
    per four tokens (ragged last group; rows of x that start on odd 2-byte
    boundaries when the width is odd): every token must come out as if it were
    walked alone, i.e. equal to the oracle to the bit, accumulated onto what y
    held."""
    sub1, op = gpu
    c = dev_case(oracle, height, width, p0, seed=7 * height + width + tokens)
    pm = op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    rng = np.random.default_rng(tokens)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
    pre = so.f32_to_bf16_bits(rng.standard_normal((tokens, height)).astype(np.float32))
    y = bf16_dev(pre).clone()
    pm.matvec_tokens(bf16_dev(xs), y)
    got = bits_host(y)
    for i in list(range(0, tokens, 23)) + list(range(tokens - 5, tokens)):
        want = oracle.matvec_gap(c['codes'], c['row_off'], c['mm'], xs[i], y=pre[i])
        assert np.array_equal(got[i], want), i
    # all tokens, one launch each for a few and in small batches for the rest
    # (the per-token kernels)
    y1 = bf16_dev(pre).clone()
    xd = bf16_dev(xs)
    for lo in range(0, tokens, 16):
        pm.matvec_tokens(xd[lo:lo + 16], y1[lo:lo + 16])
    assert torch.equal(y1, y)


def test_prepared_paths_on_random_shapes(gpu, oracle):
    """Seeded random shapes, densities and token counts through the prepared
    single-matrix path (which picks among the latency kernel, the streaming
    kernel and four tokens per walk by shape and batch) and through a two-expert
    layer: sampled tokens must equal the oracle to the bit, and the stream must
    decode back to the symbols."""
    sub1, op = gpu
    from qmoe_amd import sub1_hip
    rng = np.random.default_rng(20240611)
    for trial in range(24):
        height = int(rng.integers(1, 400))
        width = int(rng.integers(1, 3000)) if trial % 3 else int(rng.integers(1, 40))
        p0 = float(rng.choice([0.0, 0.3, 0.8, 0.9, 0.97, 0.999]))
        tokens = int(rng.choice([1, 2, 3, 5, 17, 130, 600]))
        c = dev_case(oracle, height, width, p0, seed=5000 + trial)
        pm = op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
        assert np.array_equal(pm.decode().cpu().numpy(), c['t']), (trial, height, width)
        xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
        pre = so.f32_to_bf16_bits(rng.standard_normal((tokens, height)).astype(np.float32))
        y = bf16_dev(pre).clone()
        pm.matvec_tokens(bf16_dev(xs), y)
        got = bits_host(y)
        for i in sorted(set([0, tokens // 2, tokens - 1])):
            want = oracle.matvec_gap(c['codes'], c['row_off'], c['mm'], xs[i], y=pre[i])
            assert np.array_equal(got[i], want), (trial, height, width, p0, tokens, i)
    for trial in range(8):
        d_model = int(rng.integers(1, 600))
        d_ff = int(rng.integers(1, 900))
        p0 = float(rng.choice([0.3, 0.9, 0.99]))
        tokens = int(rng.choice([1, 4, 33, 300]))
        stack, wi, wo = small_stack(oracle, 2, d_model, d_ff, p0, seed=6000 + trial)
        prep = stack.prepare()
        xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, d_model)).astype(np.float32))
        route = rng.integers(-1, 2, size=tokens).astype(np.int32)
        y = prep.forward(bf16_dev(xs), torch.from_numpy(route).cuda())
        got = bits_host(y)
        for i in sorted(set([0, tokens // 2, tokens - 1])):
            e = int(route[i])
            want = xs[i] if e < 0 else oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)[0]
            assert np.array_equal(got[i], want), (trial, d_model, d_ff, p0, tokens, i)


def test_tokens_of_an_expert_walk_together(gpu, oracle):
    """A batch with many tokens per expert: the launch groups the tokens by
    expert on the GPU and walks an expert's streams once for four (or three)
    of them.  Every token must equal what it gives in a small batch, dropped
    tokens pass through, expert ids that name no expert are counted, and
    sampled tokens equal the oracle."""
    from qmoe_amd import synthetic
    experts, d_model, d_ff, tokens = 6, 200, 333, 1500
    stack, wi, wo = small_stack(oracle, experts, d_model, d_ff, 0.8, seed=8100)
    prep = stack.prepare()
    rng = np.random.default_rng(81)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, d_model)).astype(np.float32))
    # counts per expert with every remainder modulo four; expert 5 gets nothing
    route = np.concatenate([np.full(400, 0), np.full(401, 1), np.full(402, 2), np.full(283, 3),
                            np.full(1, 4), np.full(8, -1), np.full(5, experts + 3)]).astype(np.int32)
    assert route.shape[0] == tokens
    rng.shuffle(route)
    x = bf16_dev(xs)
    te = torch.from_numpy(route).cuda()
    y = prep.forward(x, te)
    assert prep.launch_faults(tokens) == (0, 5)
    for rep in range(2):
        assert torch.equal(prep.forward(x, te), y)
    small = torch.cat([prep.forward(x[lo:lo + 50].contiguous(), te[lo:lo + 50].contiguous())
                       for lo in range(0, tokens, 50)])
    assert torch.equal(y, small)
    got = bits_host(y)
    for i in range(0, tokens, 97):
        e = int(route[i])
        want = xs[i] if e < 0 or e >= experts else oracle.expert_ffn(wi[e], wo[e], xs[i], order=2)[0]
        assert np.array_equal(got[i], want), (i, e)


def test_full_size_c2048_layer_properties(gpu, oracle):
    """The benchmark's own workload (2048 experts of 6144x2080 and 2080x6144,
    one token each: 52 G weights) is too large for the oracle; what can be
    checked at full size without it: the prepared stream holds every weight of
    sampled experts (decoded back and compared with the packed codes decoded
    by the other kernel), zero activations give zero, doubling the activations
    doubles the output exactly (a power of two commutes with every rounding and
    with ReLU), the sweep agrees with the packed-layout kernel to the stated
    tolerance, and sampled tokens equal the oracle to the bit."""
    sub1, op = gpu
    from qmoe_amd import synthetic
    experts = 2048
    d_model, d_ff = synthetic.SHAPES['c2048']
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.9, seed=20231116)
    prep = stack.prepare()
    x = synthetic.activations(experts, d_model, seed=3)
    route = torch.arange(experts, dtype=torch.int32, device='cuda')
    y = prep.forward(x, route).clone()
    assert prep.launch_faults(experts) == (0, 0)
    assert torch.equal(prep.forward(torch.zeros_like(x), route), torch.zeros_like(x))
    assert torch.equal(prep.forward(x * 2, route), y * 2)
    assert close(y, stack.forward(x, route))
    xs = bits_host(x)
    got = bits_host(y)
    for e in (0, 1023, 2047):
        wi, wo = synthetic.expert_layers(stack, e)
        for proj, layer, width in ((0, wi, d_model), (1, wo, d_ff)):
            tern, _, bad = op.sub1decode(sub1.DEC[0], layer[0], layer[1], layer[2], width, want_w=False)
            assert bad == 0
            assert torch.equal(prep.decode(e, proj), tern), (e, proj)
        host = [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                for l in (wi, wo)]
        want, _ = oracle.expert_ffn(host[0], host[1], xs[e], order=2)
        assert np.array_equal(got[e], want), e

    def expert_on_host(e):
        wi, wo = synthetic.expert_layers(stack, e)
        return [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                for l in (wi, wo)]

    # the batched-decode configuration on the same layer: 64 tokens routed top-1
    # by a seeded softmax router over all 2048 experts, one grouped launch; every
    # token against the oracle's per-token result, to the bit
    tokens = 64
    x5 = synthetic.activations(tokens, d_model, seed=4)
    r5 = synthetic.softmax_router(tokens, experts, seed=5)
    y5 = prep.forward(x5, r5)
    assert prep.launch_faults(tokens) == (0, 0)
    assert close(y5, stack.forward(x5, r5))
    xs5, got5 = bits_host(x5), bits_host(y5)
    for t in range(tokens):
        host = expert_on_host(int(r5[t]))
        want, _ = oracle.expert_ffn(host[0], host[1], xs5[t], order=2)
        assert np.array_equal(got5[t], want), (t, int(r5[t]))
    # and batch 1: one token to one seeded uniform-random expert
    g = torch.Generator().manual_seed(6)
    one = torch.randint(0, experts, (1,), generator=g).to(torch.int32).cuda()
    y1 = prep.forward(x5[:1].contiguous(), one)
    host = expert_on_host(int(one[0]))
    want, _ = oracle.expert_ffn(host[0], host[1], xs5[0], order=2)
    assert np.array_equal(bits_host(y1)[0], want)


def test_full_size_large128_layer(gpu, oracle):
    """The Switch-large-128 layer at full size: 128 experts of 4096x1024 and
    1024x4096 with P(0) = 0.88, one token per expert.  Both kernels repeat their
    results, agree within the tolerance, sampled tokens equal the oracle to the
    bit in each kernel's own order of additions, and the prepared stream of a
    sampled expert decodes back to its symbols."""
    sub1, op = gpu
    from qmoe_amd import synthetic
    experts = 128
    d_model, d_ff = synthetic.SHAPES['large']
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.88, seed=77)
    prep = stack.prepare()
    x = synthetic.activations(experts, d_model, seed=78)
    route = torch.arange(experts, dtype=torch.int32, device='cuda')
    y_ref = stack.forward(x, route).clone()
    y_prep = prep.forward(x, route).clone()
    assert prep.launch_faults(experts) == (0, 0)
    assert close(y_prep, y_ref)
    assert torch.equal(prep.forward(x, route), y_prep)
    xs = bits_host(x)
    for e in (0, 41, 127):
        wi, wo = synthetic.expert_layers(stack, e)
        host = [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                for l in (wi, wo)]
        for got, order in ((y_ref, 1), (y_prep, 2)):
            want, _ = oracle.expert_ffn(host[0], host[1], xs[e], order=order)
            assert np.array_equal(bits_host(got[e]), want), (e, order)
    wi, wo = synthetic.expert_layers(stack, 41)
    for proj, layer, width in ((0, wi, d_model), (1, wo, d_ff)):
        tern, _, bad = op.sub1decode(sub1.DEC[0], layer[0], layer[1], layer[2], width, want_w=False)
        assert bad == 0 and torch.equal(prep.decode(41, proj), tern)


def test_rows_of_very_different_lengths_at_c2048_shapes(gpu, oracle):
    """Weights that are not iid: every row with its own share of zeros between
    75% and 98%, one row in a hundred all zero and one in a hundred without a
    zero (synthetic.ROWS), at the Switch-c-2048 shapes.  Rows from 0 to 6144
    non-zeros share the row order and the slices of one matrix; the stream
    must still hold every weight (decoded back against the symbols it was made
    from) and every token must equal the oracle to the bit, in the batch sizes
    that pick the different kernels."""
    sub1, op = gpu
    from qmoe_amd import synthetic
    experts = 5
    d_model, d_ff = synthetic.SHAPES['c2048']
    stack, wi_sym, wo_sym = synthetic.build_stack(experts, d_model, d_ff, synthetic.ROWS, seed=31337,
                                                  keep_symbols=True)
    # the statistics asked for are there: empty rows, rows without a zero, and all in between
    nz = (wo_sym[0] != 0).sum(1)
    assert int((nz == 0).sum()) > 0 and int((nz == d_ff).sum()) > 0
    assert int(((nz > 0.02 * d_ff) & (nz < 0.25 * d_ff)).sum()) > 0.9 * d_model
    prep = stack.prepare()
    for e in range(experts):
        assert torch.equal(prep.decode(e, 0), wi_sym[e]), e
        assert torch.equal(prep.decode(e, 1), wo_sym[e]), e
    walked, in_rows = prep.entry_counts()
    assert 0 < in_rows <= walked

    def expert_on_host(e):
        wi, wo = synthetic.expert_layers(stack, e)
        return [tuple(bits_host(t) if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                for l in (wi, wo)]

    hosts = [expert_on_host(e) for e in range(experts)]
    kernels = set()
    for tokens in (1, 7, 300):
        x = synthetic.activations(tokens, d_model, seed=90 + tokens)
        route = (torch.arange(tokens, dtype=torch.int32, device='cuda') * 3 + 1) % experts
        y = prep.forward(x, route)
        kernels.add(_kernel_name())
        assert prep.launch_faults(tokens) == (0, 0)
        assert close(y, stack.forward(x, route))
        xs, got = bits_host(x), bits_host(y)
        for t in sorted({0, tokens // 2, tokens - 1}):
            e = int(route[t])
            want, _ = oracle.expert_ffn(hosts[e][0], hosts[e][1], xs[t], order=2)
            assert np.array_equal(got[t], want), (tokens, t, e)
    assert len(kernels) >= 2, kernels


def _kernel_name():
    from qmoe_amd import _lib
    return _lib.load().sub1_last_kernel().decode()
