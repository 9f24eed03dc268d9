"""Many tokens through one matrix on the matrix cores (the tile form and
matvec_tiles_kernel): the tile form must hold every weight (decoded back,
bit-exact against the oracle's decode of the codes), and the products must lie
within the fp32 error bound of the double-precision product and within the
stated 1e-2 of the reference kernel's lane-order arithmetic.  Bit-equality with
the row-walking kernels is not claimed: the matrix cores add in their own
order."""
import numpy as np
import pytest
import torch

from oracle import sub1_oracle as so
from test_gpu_parity import REL_TOL, bf16_dev, bits_host, dev_case

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def gpu():
    from qmoe_amd import sub1, sub1_hip
    assert torch.cuda.is_available() and sub1.DEC
    return sub1, sub1_hip


def check_tokens(oracle, c, xs, pre, got, rows):
    """Tokens `rows` of the launch against the oracle: error bound against the
    double-precision product, 1e-2 against the lane-order result, on top of
    what y held before."""
    for i in rows:
        exact, sum_abs = oracle.matvec_f64(c['t'].astype(np.uint8), c['mm'], xs[i])
        # y_new = bf16(y_old + bf16(res)): two bf16 roundings and the fp32 sum's own error
        y_old = so.bf16_bits_to_f32(pre[i]).astype(np.float64)
        y = so.bf16_bits_to_f32(got[i]).astype(np.float64)
        bound = (2.0 ** -8 * np.abs(exact) + 64 * 2.0 ** -24 * sum_abs
                 + 2.0 ** -8 * np.abs(y_old + exact) + 1e-30)
        assert np.all(np.abs(y - (y_old + exact)) <= bound), i
        lanes = so.bf16_bits_to_f32(oracle.matvec_lanes(c['codes'], c['row_off'], c['mm'], xs[i],
                                                        y=pre[i])).astype(np.float64)
        assert np.linalg.norm(y - lanes) <= REL_TOL * max(np.linalg.norm(lanes), 1e-30), i


def check_all_tokens(oracle, c, xs, pre, got):
    """Every token of the launch against the double-precision product of the
    decoded matrix (numpy, not the kernel's arithmetic): the same bound as in
    check_tokens."""
    w = so.bf16_bits_to_f32(oracle.dequant(c['t'].astype(np.uint8), c['mm'])).astype(np.float64)
    x = so.bf16_bits_to_f32(xs).astype(np.float64)
    exact, sum_abs = x @ w.T, np.abs(x) @ np.abs(w).T
    y_old = so.bf16_bits_to_f32(pre).astype(np.float64)
    y = so.bf16_bits_to_f32(got).astype(np.float64)
    bound = (2.0 ** -8 * np.abs(exact) + 64 * 2.0 ** -24 * sum_abs
             + 2.0 ** -8 * np.abs(y_old + exact) + 1e-30)
    worst = np.abs(y - (y_old + exact)) - bound
    assert np.all(worst <= 0), np.unravel_index(np.argmax(worst), worst.shape)


@pytest.mark.parametrize('height,width,p0,tokens', [
    (3072, 768, 0.9, 568), (768, 3072, 0.9, 200), (4096, 1024, 0.88, 64), (1024, 4096, 0.88, 129),
    (6144, 2080, 0.9, 70), (2080, 6144, 0.9, 65), (2080, 6144, 0.9, 300),
    (77, 333, 0.7, 100),          # ragged rows, columns and tokens; odd width: x rows unaligned
    (130, 15, 0.3, 64), (1, 4000, 0.95, 3), (200, 129, 0.0, 67), (64, 128, 0.5, 1)])
def test_tiles_product(gpu, oracle, height, width, p0, tokens):
    sub1, op = gpu
    c = dev_case(oracle, height, width, p0, seed=11 * height + width + tokens)
    tm = op.TiledMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    # the copy holds every weight
    assert np.array_equal(tm.decode().cpu().numpy(), c['t'].astype(np.uint8))
    rng = np.random.default_rng(tokens + width)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
    pre = so.f32_to_bf16_bits(rng.standard_normal((tokens, height)).astype(np.float32))
    y = bf16_dev(pre).clone()
    tm.matvec_tokens(bf16_dev(xs), y)
    got = bits_host(y)
    rows = sorted(set(list(range(0, tokens, 41)) + [tokens - 1, min(63, tokens - 1),
                                                    min(64, tokens - 1)]))
    check_tokens(oracle, c, xs, pre, got, rows)
    check_all_tokens(oracle, c, xs, pre, got)
    # the same launch again gives the same bits, and so does any split of the
    # tokens into launches (a token's result does not depend on its tile mates)
    y2 = bf16_dev(pre).clone()
    tm.matvec_tokens(bf16_dev(xs), y2)
    assert torch.equal(y, y2)
    y3 = bf16_dev(pre).clone()
    xd = bf16_dev(xs)
    for lo in range(0, tokens, 50):
        tm.matvec_tokens(xd[lo:lo + 50].contiguous(), y3[lo:lo + 50])
    assert torch.equal(y, y3)
    # agreement with the row-walking kernel on the prepared stream, to rounding
    if width <= op.PREPARED_MAX_WIDTH:
        pm = op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
        y4 = bf16_dev(pre).clone()
        pm.matvec_tokens(xd, y4)
        a, b = y.float().double(), y4.float().double()
        assert torch.linalg.norm(a - b) <= REL_TOL * torch.linalg.norm(b)


@pytest.mark.parametrize('height,width,p0,tokens,blocks_of', [
    (3072, 768, 0.9, 700, 64),       # windows split two ways, rows in groups of 128
    (4096, 1024, 0.88, 1100, 64),    # one part, rows in groups of 256
    (3200, 2080, 0.9, 1500, 64),     # 50 blocks of rows (not a multiple of four), a ragged last window
    (6272, 520, 0.9, 2100, 128)])    # blocks of 128 tokens, the last with 52
def test_long_sequences_share_their_activations(gpu, oracle, height, width, p0, tokens, blocks_of):
    """From the number of tokens on at which the one-wavefront workgroups no
    longer fit the chip at once, workgroups of four wavefronts share each window
    of activations (matvec_tiles_shared_kernel).  Every token against the
    double-precision product; and the same bits as the same tokens in launches
    short enough for the other kernel (same sums in the same order), which also
    shows that a token's result does not depend on the launch."""
    sub1, op = gpu
    from qmoe_amd import _lib
    c = dev_case(oracle, height, width, p0, seed=7 * height + width + tokens)
    tm = op.TiledMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    rng = np.random.default_rng(tokens + width)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
    pre = so.f32_to_bf16_bits(rng.standard_normal((tokens, height)).astype(np.float32))
    xd = bf16_dev(xs)
    y = bf16_dev(pre).clone()
    tm.matvec_tokens(xd, y)
    assert _lib.load().sub1_last_kernel() == b'matvec_tiles_shared_kernel<%d>' % blocks_of
    check_all_tokens(oracle, c, xs, pre, bits_host(y))
    check_tokens(oracle, c, xs, pre, bits_host(y), [0, tokens // 2, tokens - 1])
    y2 = bf16_dev(pre).clone()
    tm.matvec_tokens(xd, y2)
    assert torch.equal(y, y2)
    y3 = bf16_dev(pre).clone()
    for lo in range(0, tokens, 200):
        tm.matvec_tokens(xd[lo:lo + 200].contiguous(), y3[lo:lo + 200])
        assert _lib.load().sub1_last_kernel() == b'matvec_tiles_kernel'
    assert torch.equal(y, y3)
    # rows of y and x further apart than they are long
    xw = torch.zeros((tokens, width + 24), dtype=torch.bfloat16, device='cuda')
    xw[:, :width] = xd
    yw = torch.zeros((tokens, height + 6), dtype=torch.bfloat16, device='cuda')
    yw[:, :height] = bf16_dev(pre)
    yw[:, height:] = 7.0
    import ctypes
    _lib.check(_lib.load().sub1_matvec_tiles(
        ctypes.byref(tm._c), 0, xw.data_ptr(), width + 24, yw.data_ptr(), height + 6, tokens,
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    assert _lib.load().sub1_last_kernel().startswith(b'matvec_tiles_shared_kernel')
    assert torch.equal(yw[:, :height], y) and bool((yw[:, height:] == 7.0).all())


def test_both_tile_kernels_give_the_same_bits_on_any_shape(gpu, oracle):
    """Random shapes (blocks of rows that are no multiple of a workgroup's,
    fewer windows than parts, ragged last windows, a last block of tokens with
    one token or with 127): the kernel whose workgroups share their activations,
    with blocks of 64 and of 128 tokens, against the one-wavefront kernel, bit
    for bit, and every token against the double-precision product."""
    sub1, op = gpu
    from qmoe_amd import _lib
    lib = _lib.load()
    rng = np.random.default_rng(2024)
    shapes = [(2, 8, 1), (64, 128, 64), (66, 136, 65), (256, 128, 129), (258, 1032, 127), (640, 264, 200)]
    shapes += [(2 * int(rng.integers(1, 400)), 8 * int(rng.integers(1, 200)), int(rng.integers(1, 330)))
               for _ in range(14)]
    try:
        for n, (height, width, tokens) in enumerate(shapes):
            c = dev_case(oracle, height, width, float(rng.uniform(0.3, 0.97)), seed=500 + n)
            tm = op.TiledMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
            xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
            pre = so.f32_to_bf16_bits(rng.standard_normal((tokens, height)).astype(np.float32))
            xd = bf16_dev(xs)
            outs = []
            for which, name in ((1, b'matvec_tiles_kernel'), (2, b'matvec_tiles_shared_kernel<64>'),
                                (3, None)):
                _lib.check(lib.sub1_test_tiles_kernel(which))
                y = bf16_dev(pre).clone()
                tm.matvec_tokens(xd, y)
                if name:
                    assert lib.sub1_last_kernel() == name, (height, width, tokens)
                else:
                    assert lib.sub1_last_kernel().startswith(b'matvec_tiles_shared_kernel')
                outs.append(y)
            assert torch.equal(outs[0], outs[1]), (height, width, tokens)
            assert torch.equal(outs[0], outs[2]), (height, width, tokens)
            check_all_tokens(oracle, c, xs, pre, bits_host(outs[0]))
    finally:
        _lib.check(lib.sub1_test_tiles_kernel(0))
    assert lib.sub1_test_tiles_kernel(4) != 0


def test_tiles_closed_forms(gpu, oracle):
    """Unit vectors pick a column exactly; zero activations leave y as it was;
    doubling the activations doubles the product exactly (y zero before)."""
    sub1, op = gpu
    height, width, tokens = 96, 300, 70
    c = dev_case(oracle, height, width, 0.6, seed=4321)
    tm = op.TiledMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    w = so.bf16_bits_to_f32(oracle.dequant(c['t'].astype(np.uint8), c['mm']))
    one = so.f32_to_bf16_bits(np.array([1.0], np.float32))[0]
    xs = np.zeros((tokens, width), dtype=np.uint16)
    cols = [(7 * i) % width for i in range(tokens)]
    for i, k in enumerate(cols):
        xs[i, k] = one
    y = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
    tm.matvec_tokens(bf16_dev(xs), y)
    got = so.bf16_bits_to_f32(bits_host(y))
    for i, k in enumerate(cols):
        assert np.array_equal(got[i], w[:, k]), (i, k)
    pre = so.f32_to_bf16_bits(np.random.default_rng(1).standard_normal((tokens, height)).astype(np.float32))
    y = bf16_dev(pre).clone()
    tm.matvec_tokens(torch.zeros((tokens, width), dtype=torch.bfloat16, device='cuda'), y)
    assert np.array_equal(bits_host(y), pre)
    x = torch.randn((tokens, width), generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    y1 = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
    y2 = torch.zeros_like(y1)
    tm.matvec_tokens(x, y1)
    tm.matvec_tokens(x * 2, y2)
    assert torch.equal(y2, y1 * 2)


def test_tiles_matrix_set_and_arguments(gpu, oracle):
    """Several matrices in one tile buffer; arguments are checked."""
    sub1, op = gpu
    from qmoe_amd._lib import Sub1Error
    height, width, count, tokens = 130, 200, 3, 80
    cases = [dev_case(oracle, height, width, 0.8, seed=650 + i) for i in range(count)]
    tm = op.TiledMatrix(sub1.DEC[0], [c['w_comp'] for c in cases], [c['row_off_d'] for c in cases],
                        [c['mm_d'] for c in cases], width)
    rng = np.random.default_rng(9)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
    pre = np.zeros((tokens, height), dtype=np.uint16)
    for m, c in enumerate(cases):
        assert np.array_equal(tm.decode(m).cpu().numpy(), c['t'].astype(np.uint8))
        y = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
        tm.matvec_tokens(bf16_dev(xs), y, matrix=m)
        check_tokens(oracle, c, xs, pre, bits_host(y), [0, 63, 64, 79])
    y = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
    with pytest.raises(Sub1Error):
        tm.matvec_tokens(bf16_dev(xs), y, matrix=3)
    with pytest.raises(ValueError):
        tm.matvec_tokens(bf16_dev(xs)[:, :-1].contiguous(), y)
    bad = cases[0]['row_off_d'].clone()
    bad[40] -= 1
    with pytest.raises(Sub1Error):
        op.TiledMatrix(sub1.DEC[0], cases[0]['w_comp'], bad, cases[0]['mm_d'], width)


def test_sub1linear_takes_the_tiles_from_64_tokens_on(gpu, oracle):
    """Sub1Linear.forward on a sequence: the tile form from `tile_tokens` tokens
    on, the prepared stream below (the same bits for a token whatever its
    batch), the packed buffers for one or two tokens on request; all within the
    tolerance of the dense product, and the tile copy follows the buffers like
    the prepared one."""
    sub1, op = gpu
    from qmoe_amd import _lib
    t, mm = so.synthetic_ternary(320, 512, 0.85, seed=77)
    w = bf16_dev(oracle.dequant(t.astype(np.uint8), mm))
    lin = sub1.Sub1Linear.make(w)
    x = torch.randn((100, 512), generator=torch.Generator().manual_seed(3)).bfloat16().cuda()
    ref = x.float() @ w.float().t()
    y = lin(x)
    assert _lib.load().sub1_last_kernel() .startswith(b'matvec_tiles_')
    assert torch.linalg.norm(y.float() - ref) <= REL_TOL * torch.linalg.norm(ref)
    y_few = lin(x[:10])
    assert not _lib.load().sub1_last_kernel().startswith(b'matvec_tiles_')
    assert torch.linalg.norm(y_few.float() - ref[:10]) <= REL_TOL * torch.linalg.norm(ref[:10])
    # below the tile form a token's bits do not depend on the tokens it comes with
    for n in (1, 2, 3, 63):
        assert torch.equal(lin(x[:n]), lin(x[:63])[:n]), n
    # on request one or two tokens go straight from the packed buffers, a wavefront per row
    lin.packed_tokens = 2
    y_two = lin(x[:2])
    assert _lib.load().sub1_last_kernel() == b'matvec_wave_kernel<4>'
    assert torch.linalg.norm(y_two.float() - ref[:2]) <= REL_TOL * torch.linalg.norm(ref[:2])
    # and long sequences stay on the prepared stream, to the bit, where the tile form is switched off
    lin.packed_tokens, lin.tile_tokens = 0, None
    assert torch.equal(lin(x)[:63], lin(x[:63]))
    assert not _lib.load().sub1_last_kernel().startswith(b'matvec_tiles_')
    lin.tile_tokens = 64
    lin.ter_minmax = (lin.ter_minmax.float() * 2).bfloat16()
    assert torch.equal(lin(x).float(), 2 * y.float())


def test_tiles_multiply_zero_weights_like_the_reference(gpu, oracle):
    """An infinite activation: the matrix cores multiply a zero weight by it
    like any other (0 x inf = NaN, which is what reference
    sub1_cuda_kernel.cu:190 computes too), so no row of that token stays
    finite; the row-walking kernels leave the rows that have no weight in the
    column as they would be with a zero there.  Other tokens are untouched."""
    sub1, op = gpu
    height, width, tokens, col = 128, 256, 66, 37
    c = dev_case(oracle, height, width, 0.8, seed=8080)
    rng = np.random.default_rng(5)
    xs = so.f32_to_bf16_bits(rng.standard_normal((tokens, width)).astype(np.float32))
    clean = xs.copy()
    clean[3, col] = 0
    xs[3, col] = 0x7f80                      # +inf
    tm = op.TiledMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    y_inf = torch.zeros((tokens, height), dtype=torch.bfloat16, device='cuda')
    y_clean = torch.zeros_like(y_inf)
    tm.matvec_tokens(bf16_dev(xs), y_inf)
    tm.matvec_tokens(bf16_dev(clean), y_clean)
    assert not torch.isfinite(y_inf[3].float()).any()
    others = [i for i in range(tokens) if i != 3]
    assert torch.equal(y_inf[others], y_clean[others])
    pm = op.PreparedMatrix(sub1.DEC[0], c['w_comp'], c['row_off_d'], c['mm_d'], width)
    w_inf = torch.zeros_like(y_inf)
    w_clean = torch.zeros_like(y_inf)
    pm.matvec_tokens(bf16_dev(xs), w_inf)
    pm.matvec_tokens(bf16_dev(clean), w_clean)
    no_weight = torch.from_numpy(c['t'][:, col] == 0).cuda()
    assert no_weight.any() and (~no_weight).any()
    assert torch.equal(w_inf[3][no_weight], w_clean[3][no_weight])
    assert not torch.isfinite(w_inf[3][~no_weight].float()).any()
    assert torch.equal(w_inf[others], w_clean[others])
