"""Benchmark of the compressed-expert hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the grouped expert launch over one batch of synthetic
tokens.  The default workload is the Switch-c-2048 MoE layer swept with one
token per expert (2048 experts, wi 6144x2080 and wo 2080x6144 each, about
4.6 GB of compressed weights: larger than every cache, so the rate is an HBM
rate).  Prints ONE JSON line: microseconds per layer, the achieved rate on
algorithmic (compressed) bytes against the 8 TB/s HBM peak, and the CPU
oracle timed on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant kernel.  A recorded figure, not measured by this run:
# it comes from rocprofv3 counter runs of this same command (FETCH_SIZE x 2.0 + WRITE_SIZE x
# 1.0, the factors a 1 GiB device copy reads on those counters), summarised in the file
# named beside it (the copy of known size is part of `--sweep-only`).  None where no such
# run was made.
MEASURED_TRAFFIC = {'c2048-sweep': (4.884e9 + 0.009e9,
                                    'profiles/moe_prepared_fused_kernel_c2048_sweep.txt')}

WORKLOADS = {
    # name: (shape key, experts, p_zero, description)
    'c2048-sweep': ('c2048', 2048, 0.90,
                    'Switch-c-2048 MoE layer, 2048 experts, 1 token per expert (sweep)'),
    'large128': ('large', 128, 0.88, 'Switch-large-128 MoE layer, 1 token per expert'),
    'base128': ('base', 128, 0.90, 'Switch-base-128 MoE layer, 1 token per expert'),
}


def algorithmic_bytes(stack, experts_used):
    """Bytes the products of one launch have to read and write, on the
    reference's compressed layout (per product: 2*codes + 4*(H+1) row offsets +
    4*H min/max + 2*W input + 2*H output)."""
    total = 0
    for e in experts_used:
        total += 2 * int(stack.wi_codes[e]) + 2 * int(stack.wo_codes[e])
        for h, w in ((stack.d_ff, stack.d_model), (stack.d_model, stack.d_ff)):
            total += 4 * (h + 1) + 4 * h + 2 * w + 2 * h
    return total


def rel_diff(a, b):
    """Normwise relative difference of two bf16 results (the kernels on the
    packed layout and on the prepared stream add in different orders)."""
    import torch
    a, b = a.float().double(), b.float().double()
    return float('%.3g' % (torch.linalg.norm(a - b) / torch.linalg.norm(b)).item())


PREHEAT_S = 0.1


def time_launches(fn, steps, warmup, stream_ptr, preheat_s=PREHEAT_S):
    """(wall seconds for `steps` calls, average microseconds per call from HIP
    events recorded on the launch stream).  Before the `warmup` untimed calls
    the same call is repeated, untimed, for `preheat_s` seconds: from idle the
    GPU takes about 40 ms of load to reach its clocks (the c-2048 sweep reads
    1250 us in its first ten launches, 1000 us from the fortieth on), and a
    short warm-up would time that ramp instead of the kernel."""
    import ctypes
    import torch
    from qmoe_amd import _lib
    lib = _lib.load()
    tick = time.perf_counter()
    while time.perf_counter() - tick < preheat_s:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    tick = time.perf_counter()
    _lib.check(lib.sub1_timing_begin(stream_ptr))
    for _ in range(steps):
        fn()
    us = ctypes.c_double()
    _lib.check(lib.sub1_timing_end(stream_ptr, ctypes.byref(us)))
    torch.cuda.synchronize()
    wall = time.perf_counter() - tick
    return wall, us.value / steps


def cpu_baseline(stack, x, sample_experts, threads, budget_s=10.0):
    """The CPU oracle's reference-order decode+matvec (a scalar C port of the
    reference kernel's arithmetic) on the first experts of the same stack:
    `threads` experts at a time on as many host cores (the C call runs outside
    the interpreter lock).  Returns (experts done, wall seconds inside the
    oracle); transfers of the experts to the host are not timed."""
    import concurrent.futures
    import numpy as np
    import torch
    from oracle import sub1_oracle as so
    from qmoe_amd import synthetic
    o = so.COracle()
    o.tables()
    done, spent = 0, 0.0
    with concurrent.futures.ThreadPoolExecutor(max_workers=threads) as pool:
        while done < sample_experts and spent < budget_s:
            batch = []
            for e in range(done, min(done + 4 * threads, sample_experts)):
                wi, wo = synthetic.expert_layers(stack, e)
                host = [tuple(t.view(torch.int16).cpu().numpy().view(np.uint16)
                              if t.dtype != torch.int32 else t.cpu().numpy() for t in l)
                        for l in (wi, wo)]
                batch.append((host[0], host[1],
                              x[e].view(torch.int16).cpu().numpy().view(np.uint16)))
            tick = time.perf_counter()
            list(pool.map(lambda b: o.expert_ffn(b[0], b[1], b[2], order=0), batch))
            spent += time.perf_counter() - tick
            done += len(batch)
    return done, spent


def cpu_single_matrix_us(seed):
    """The first configuration of the list: one Switch-base wi matrix
    (3072 x 768, P(0) = 0.9), one token, decode + product on one host core
    through the C oracle in the reference kernel's arithmetic.  Microseconds
    per product."""
    from oracle import sub1_oracle as so
    o = so.COracle()
    o.tables()
    t, mm = so.synthetic_ternary(3072, 768, 0.9, seed)
    codes, row_off = o.encode(t)
    xv = so.synthetic_activation(768, seed + 1)
    o.matvec_lanes(codes, row_off, mm, xv)
    reps = 20
    tick = time.perf_counter()
    for _ in range(reps):
        o.matvec_lanes(codes, row_off, mm, xv)
    return (time.perf_counter() - tick) / reps * 1e6


def cpu_python_decode_matmul_us(seed):
    """The reference's own host path for the first configuration
    (test.py:103-115 and :180): the codes of a 3072 x 768 matrix expanded to
    dense values in interpreted Python through the entry strings, then one
    bf16 torch.matmul on the host.  Microseconds for the pair; nearly all of
    it is the expansion."""
    import torch
    from oracle import sub1_oracle as so
    o = so.COracle()
    o.tables()
    entries, _ = o.entries()
    t, mm = so.synthetic_ternary(3072, 768, 0.9, seed)
    codes, row_off = o.encode(t)
    xv = torch.from_numpy(so.bf16_bits_to_f32(so.synthetic_activation(768, seed + 1))).to(torch.bfloat16)
    levels = so.bf16_bits_to_f32(mm).reshape(-1, 2)
    tick = time.perf_counter()
    dense = []
    for r in range(3072):
        lo, hi = float(levels[r, 0]), float(levels[r, 1])
        table = (0.0, lo, hi)
        dense.extend(table[s] for s in so.expand_codes(codes[row_off[r]:row_off[r + 1]], entries, 768))
    w = torch.tensor(dense, dtype=torch.float32).reshape(3072, 768).to(torch.bfloat16)
    y = torch.matmul(w, xv)
    spent = time.perf_counter() - tick
    want = so.bf16_bits_to_f32(o.matvec_lanes(codes, row_off, mm, so.synthetic_activation(768, seed + 1)))
    err = float((y.float() - torch.from_numpy(want)).norm() / torch.from_numpy(want).norm())
    assert err < 1e-2, 'python decode + matmul differs from the C oracle by %g' % err
    return spent * 1e6


def dense_gemv_us(stack, x, experts):
    """Dense bf16 batched GEMV (torch.bmm -> hipBLASLt/rocBLAS) on the decoded
    weights of the first `experts` experts, microseconds per expert FFN."""
    import torch
    from qmoe_amd import sub1_hip, synthetic
    wis, wos = [], []
    for e in range(experts):
        wi, wo = synthetic.expert_layers(stack, e)
        wis.append(sub1_hip.sub1decode(stack.dec, wi[0], wi[1], wi[2], stack.d_model,
                                       want_tern=False)[1])
        wos.append(sub1_hip.sub1decode(stack.dec, wo[0], wo[1], wo[2], stack.d_ff,
                                       want_tern=False)[1])
    wi = torch.stack(wis)
    wo = torch.stack(wos)
    del wis, wos
    xv = x[:experts].unsqueeze(2).contiguous()

    def run():
        h = torch.relu(torch.bmm(wi, xv))
        return torch.bmm(wo, h)

    for _ in range(3):
        run()
    torch.cuda.synchronize()
    tick = time.perf_counter()
    reps = 10
    for _ in range(reps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - tick) / reps / experts * 1e6


def single_matrix_protocol(seed, stream_ptr):
    """The reference's own benchmark (test.py:117-126 and 163-186: 100 warm-up
    + 1000 calls of one product per Switch shape, compressed against dense
    bf16 torch.matmul) with one token.  Per shape: kernel-side microseconds
    from HIP events over back-to-back calls for the prepared layout, the
    packed layout (`sub1matvec`, the drop-in call) and the dense product, and
    the reference's wall-clock protocol (synchronise after every call) for the
    drop-in call and the dense product.  Plus 568 tokens through the same
    matrix in one launch (walking the prepared stream once per four tokens, and
    on the matrix cores from the tile form), against the dense GEMM."""
    import torch
    from qmoe_amd import sub1, sub1_hip, synthetic

    def sync_each_us(fn, warmup=100, reps=1000):
        for _ in range(warmup):
            fn()
            torch.cuda.synchronize()
        tick = time.perf_counter()
        for _ in range(reps):
            fn()
            torch.cuda.synchronize()
        return (time.perf_counter() - tick) / reps * 1e6

    g = torch.Generator(device='cuda')
    g.manual_seed(seed)
    dec, trie = sub1.device_tables('cuda:0')
    rows = {}
    for name, (h, w, p0) in (('base_wi', (3072, 768, 0.9)), ('base_wo', (768, 3072, 0.9)),
                             ('large_wi', (4096, 1024, 0.88)), ('large_wo', (1024, 4096, 0.88)),
                             ('c2048_wi', (6144, 2080, 0.9)), ('c2048_wo', (2080, 6144, 0.9))):
        t = synthetic.draw_symbols(h, w, p0, g, 'cuda')
        mm = synthetic.draw_minmax(h, g, 'cuda')
        lut = torch.stack((torch.zeros(h, device='cuda', dtype=torch.bfloat16), mm[0::2], mm[1::2]), 1)
        dense = torch.gather(lut, 1, t.long()).contiguous()
        row_off = torch.zeros(h + 1, dtype=torch.int32, device='cuda')
        w_comp = sub1_hip.sub1pack(trie, t, row_off)
        del t
        x = torch.randn(w, generator=g, device='cuda').bfloat16()
        y = torch.zeros(h, dtype=torch.bfloat16, device='cuda')
        x2, y2 = x.reshape(1, -1), torch.zeros((1, h), dtype=torch.bfloat16, device='cuda')
        xd, yd = x.reshape(-1, 1), torch.zeros((h, 1), dtype=torch.bfloat16, device='cuda')
        pm = sub1_hip.PreparedMatrix(dec, w_comp, row_off, mm, w)
        packed = lambda: sub1_hip.sub1matvec(dec, w_comp, row_off, mm, x, y)
        matmul = lambda: torch.matmul(dense, xd, out=yd)
        rows[name] = {
            'prepared_us': round(time_launches(lambda: pm.matvec_tokens(x2, y2), 1000, 100, stream_ptr)[1], 2),
            'packed_us': round(time_launches(packed, 1000, 100, stream_ptr)[1], 2),
            'dense_bf16_us': round(time_launches(matmul, 1000, 100, stream_ptr)[1], 2),
            'sync_each_packed_us': round(sync_each_us(packed), 2),
            'sync_each_dense_us': round(sync_each_us(matmul), 2),
            'compressed_bytes': 2 * w_comp.numel(), 'dense_bytes': 2 * h * w,
            # the ratio reference test.py:178 prints: 16 bits per weight against the
            # codes plus 64 bits per row of offsets and min/max
            'reference_compression_ratio': round(
                16.0 * h * w / (16.0 * w_comp.numel() + 64.0 * (h + 1)), 3)}
        # a sequence through the same layer (the encoder side): 568 tokens in one
        # launch, the stream walked once per four tokens, against a dense bf16 GEMM
        xt = torch.randn((568, w), generator=g, device='cuda').bfloat16()
        yt = torch.zeros((568, h), dtype=torch.bfloat16, device='cuda')
        ydt = torch.zeros((h, 568), dtype=torch.bfloat16, device='cuda')
        xdt = xt.t().contiguous()
        rows[name]['tokens568_prepared_us'] = round(
            time_launches(lambda: pm.matvec_tokens(xt, yt), 100, 10, stream_ptr)[1], 2)
        # the same 568 tokens on the matrix cores from the tile form (what
        # Sub1Linear.forward uses from 64 tokens on): weights decoded once per 64 tokens
        tm = sub1_hip.TiledMatrix(dec, w_comp, row_off, mm, w)
        rows[name]['tokens568_tiles_us'] = round(
            time_launches(lambda: tm.matvec_tokens(xt, yt), 100, 10, stream_ptr)[1], 2)
        rows[name]['tiles_bytes'] = int(tm.entries.numel() + tm.meta.numel())
        rows[name]['tokens568_dense_bf16_us'] = round(
            time_launches(lambda: torch.matmul(dense, xdt, out=ydt), 100, 10, stream_ptr)[1], 2)
        # longer sequences (two and four of those): from the length at which the
        # tile kernel's workgroups no longer fit the chip at once, workgroups
        # that share their activations take over
        for tokens in (1136, 2272):
            xl = torch.randn((tokens, w), generator=g, device='cuda').bfloat16()
            yl = torch.zeros((tokens, h), dtype=torch.bfloat16, device='cuda')
            ydl = torch.zeros((h, tokens), dtype=torch.bfloat16, device='cuda')
            xdl = xl.t().contiguous()
            rows[name]['tokens%d_tiles_us' % tokens] = round(
                time_launches(lambda: tm.matvec_tokens(xl, yl), 100, 10, stream_ptr)[1], 2)
            rows[name]['tokens%d_dense_bf16_us' % tokens] = round(
                time_launches(lambda: torch.matmul(dense, xdl, out=ydl), 100, 10, stream_ptr)[1], 2)
    return rows


def faster_mlp_protocol(stack, seed, stream_ptr, tokens=64):
    """The sparse-MLP module around the experts (reference sub1.py:299-321) on
    `tokens` tokens: router, one launch over the experts, probability scaling,
    beside the reference's own way through the same modules, a Python loop over
    the experts that received tokens with two products per token.  The router
    is transformers' SwitchTransformersTop1Router built from a config where
    transformers can be imported."""
    import types
    import torch
    import torch.nn as nn
    from qmoe_amd import sub1, synthetic
    experts, d_model, d_ff = stack.experts, stack.d_model, stack.d_ff

    class Expert(nn.Module):
        def __init__(self, wi, wo):
            super().__init__()
            self.wi, self.wo = wi, wo

        def forward(self, x):
            return self.wo(torch.relu(self.wi(x)))

    def layer(triple, height):
        lin = sub1.Sub1Linear(height, triple[0].numel())
        lin.w_comp.data, lin.row_off.data, lin.ter_minmax.data = triple
        return lin

    modules = nn.ModuleDict()
    for e in range(experts):
        wi, wo = synthetic.expert_layers(stack, e)
        modules['expert_%d' % e] = Expert(layer(wi, d_ff), layer(wo, d_model))
    try:
        from transformers import SwitchTransformersConfig
        from transformers.models.switch_transformers.modeling_switch_transformers import (
            SwitchTransformersTop1Router)
        cfg = SwitchTransformersConfig(d_model=d_model, d_ff=d_ff, num_experts=experts,
                                       expert_capacity=tokens, router_jitter_noise=0.0)
        router, which = SwitchTransformersTop1Router(cfg).cuda().eval(), 'transformers'
    except Exception as exc:                                   # absent or another layout
        return {'skipped': 'no transformers router: %s' % type(exc).__name__}
    fast = sub1.FasterMLP(types.SimpleNamespace(router=router, experts=modules),
                          router_outputs=False)
    hidden = synthetic.activations(tokens, d_model, seed).view(1, tokens, d_model)

    def loop():                      # reference sub1.py:306-321 on the same modules
        mask, probs, _ = sub1._router_outputs(router(hidden), experts)
        next_states = hidden.clone()
        for e in torch.nonzero(mask.sum(dim=(0, 1)), as_tuple=True)[0]:
            sel = mask[:, :, e].bool()
            next_states[sel] = modules['expert_%d' % int(e)](hidden[sel])
        return probs * next_states

    with torch.no_grad():
        a, b = fast(hidden), loop()
        diff = rel_diff(a, b)
        _, us_fast = time_launches(lambda: fast(hidden), 50, 5, stream_ptr)
        _, us_router = time_launches(lambda: router(hidden), 50, 5, stream_ptr)
        _, us_loop = time_launches(loop, 5, 1, stream_ptr, preheat_s=0.0)
    return {'tokens': tokens, 'router': which, 'module_us': round(us_fast, 1),
            'router_alone_us': round(us_router, 1), 'expert_loop_us': round(us_loop, 1),
            'vs_expert_loop_rel_diff': diff}


def density_sweep(seed, stream_ptr, experts=512):
    """The headline sweep at other weight statistics: the Switch-c-2048 shapes,
    `experts` experts (a stream of 1.0 to 1.9 GB, beyond every cache), a token
    per expert, at four shares of zeros and on rows whose share of zeros
    differs from row to row (synthetic.ROWS).  The dictionary stays the fixed
    one (tuned for 88.5% zeros); the prepared stream costs 7.1 bits per
    non-zero whatever the statistics, so its size follows the non-zeros while
    the compressed bytes follow the dictionary's fit."""
    import torch
    from qmoe_amd import synthetic
    d_model, d_ff = synthetic.SHAPES['c2048']
    x = synthetic.activations(experts, d_model, seed + 1)
    route = torch.arange(experts, dtype=torch.int32, device='cuda')
    y = torch.empty_like(x)
    rows = {}
    for name, p0 in (('p0_0.80', 0.80), ('p0_0.85', 0.85), ('p0_0.88', 0.88), ('p0_0.95', 0.95),
                     ('rows_0.75_to_0.98', synthetic.ROWS)):
        st = synthetic.build_stack(experts, d_model, d_ff, p0, seed)
        pr = st.prepare()
        _, us = time_launches(lambda: pr.forward(x, route, y), 30, 5, stream_ptr)
        walked, in_rows = pr.entry_counts()
        cb = st.compressed_bytes()
        rows[name] = {
            'us_per_layer': round(us, 1), 'experts': experts,
            'compressed_bytes': cb,
            'bits_per_weight': round(16.0 * st.w_comp.numel() / (2.0 * experts * d_model * d_ff), 4),
            'prepared_stream_bytes': int(pr.stream_bytes),
            'frac_on_compressed_bytes': round(cb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            'frac_on_stream_bytes': round(pr.stream_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            'padding_share_of_entries': round(1.0 - in_rows / walked, 4)}
        del st, pr
    return rows


def hbm_rate_by_rotation(name, seed, stream_ptr, copies=6):
    """A layer whose compressed stack fits the 256 MB last-level cache, timed
    from HBM all the same: `copies` different stacks of it taken in turn, so
    that more than the cache holds passes between two uses of the same bytes."""
    import torch
    from qmoe_amd import synthetic
    shp, n_e, p_z, _ = WORKLOADS[name]
    dm, df = synthetic.SHAPES[shp]
    stacks = [synthetic.build_stack(n_e, dm, df, p_z, seed + 100 + i) for i in range(copies)]
    preps = [st.prepare() for st in stacks]
    ab = sum(algorithmic_bytes(st, range(n_e)) for st in stacks) / copies
    stream = sum(int(pr.stream_bytes) for pr in preps)
    del stacks
    xs = synthetic.activations(n_e, dm, seed + 11)
    rt = torch.arange(n_e, dtype=torch.int32, device='cuda')
    ys = torch.empty_like(xs)
    turn = [0]

    def step():
        preps[turn[0] % copies].forward(xs, rt, ys)
        turn[0] += 1

    _, us = time_launches(step, 20 * copies, 2 * copies, stream_ptr)
    return {'us_per_layer_from_hbm': round(us, 2), 'stacks_rotated': copies,
            'streams_in_rotation_bytes': stream,
            'GBps_from_hbm': round(ab / us / 1e3, 1),
            'frac_from_hbm': round(ab / us / 1e3 / HBM_PEAK_GBS, 4)}


def cpu_layer_baseline(stack, x, cores):
    """The CPU oracle on a whole small layer (a token per expert): one core on
    a bounded sample, then `cores` threads, microseconds per layer each."""
    experts = stack.experts
    done1, spent1 = cpu_baseline(stack, x, min(experts, 32), 1, budget_s=2.0)
    done, spent = cpu_baseline(stack, x, experts, cores, budget_s=3.0)
    return {'one_core_us_per_layer': round(spent1 / done1 * experts * 1e6, 1),
            'one_core_sample': '%d of %d expert FFNs, %.1f s' % (done1, experts, spent1),
            'threads': cores,
            'threads_us_per_layer': round(spent / done * experts * 1e6, 1),
            'threads_sample': '%d of %d expert FFNs, %.1f s' % (done, experts, spent)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=100)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='c2048-sweep', choices=sorted(WORKLOADS))
    ap.add_argument('--experts', type=int, default=0, help='override the expert count (debugging)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline')
    ap.add_argument('--no-dense', action='store_true', help='skip the dense bf16 comparison')
    ap.add_argument('--sweep-only', action='store_true',
                    help='only the headline sweep (what a profiler run should see)')
    ap.add_argument('--small-batch-only', type=int, default=0, metavar='TOKENS',
                    help='instead of the benchmark, run the expert layer of the workload on '
                         'this many tokens (1: one token to one expert; more: softmax router) '
                         '`--steps` times, for a profiler')
    ap.add_argument('--reference-layout-only', action='store_true',
                    help='instead of the benchmark, run the sweep `--steps` times through the launch '
                         'that reads the reference\'s packed layout and decodes the dictionary in '
                         'the kernel (no preparation), for a profiler')
    ap.add_argument('--single-matrix-only', action='store_true',
                    help='instead of the benchmark, run only the one-product-per-shape protocol')
    ap.add_argument('--seed', type=int, default=20231116)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: this build has no multi-GPU path (--gpus 1 only)')
    from qmoe_amd import _lib, build as _build
    if not os.path.exists(_lib.LIB_PATH):      # uses what is built; builds only if nothing is
        _build.build_library()
    import ctypes
    import torch
    from qmoe_amd import _lib, synthetic

    if args.single_matrix_only:
        torch.cuda.set_device(0)
        stream_ptr = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        print(json.dumps({'single_matrix_1_token': single_matrix_protocol(args.seed + 30, stream_ptr)}))
        return

    shape, experts, p_zero, desc = WORKLOADS[args.workload]
    if args.experts:
        experts = args.experts
        desc += ' [reduced to %d experts]' % experts
    d_model, d_ff = synthetic.SHAPES[shape]
    torch.cuda.set_device(0)
    tick = time.perf_counter()
    stack = synthetic.build_stack(experts, d_model, d_ff, p_zero, args.seed)
    torch.cuda.synchronize()
    print('built %d experts in %.1f s, %.3f GB compressed' %
          (experts, time.perf_counter() - tick, stack.compressed_bytes() / 1e9), file=sys.stderr)

    if args.reference_layout_only:
        x = synthetic.activations(experts, d_model, args.seed + 1)
        route = torch.arange(experts, dtype=torch.int32, device='cuda')
        y = torch.empty_like(x)
        stream_ptr = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        cal = torch.zeros(2, 1 << 28, dtype=torch.int32, device='cuda')     # the copy of known size
        torch.add(cal[0], 1, out=cal[1])
        torch.cuda.synchronize()
        del cal
        _, us = time_launches(lambda: stack.forward(x, route, y), args.steps, args.warmup, stream_ptr)
        abytes = algorithmic_bytes(stack, range(experts))
        print(json.dumps({'workload': desc, 'kernel': _lib.load().sub1_last_kernel().decode(),
                          'us_per_launch': round(us, 1), 'algorithmic_bytes': abytes,
                          'compressed_bytes': stack.compressed_bytes(),
                          'frac': round(abytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}))
        return

    tick = time.perf_counter()
    prep = stack.prepare()
    torch.cuda.synchronize()
    prepare_ms = (time.perf_counter() - tick) * 1e3
    print('prepared in %.2f s: %.3f GB of interleaved gap entries (%.3f x the packed codes) + '
          '%.3f GB of position checkpoints' %
          (prepare_ms / 1e3, prep.stream_bytes / 1e9,
           prep.stream_bytes / (2.0 * stack.w_comp.numel()),
           (prep.code_bytes - prep.stream_bytes) / 1e9), file=sys.stderr)

    if args.small_batch_only:
        t = args.small_batch_only
        xs = synthetic.activations(t, d_model, args.seed + 3)
        if t == 1:
            g = torch.Generator().manual_seed(args.seed + 2)
            rs = torch.randint(0, experts, (1,), generator=g).to(torch.int32).cuda()
        else:
            rs = synthetic.softmax_router(t, experts, args.seed + 4)
        ys = torch.empty_like(xs)
        stream_ptr = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        _, us = time_launches(lambda: prep.forward(xs, rs, ys), args.steps, args.warmup, stream_ptr)
        print(json.dumps({'workload': desc, 'tokens': t, 'us_per_layer': round(us, 2)}))
        return

    x = synthetic.activations(experts, d_model, args.seed + 1)
    route = torch.arange(experts, dtype=torch.int32, device='cuda')
    y = torch.empty_like(x)
    stream_ptr = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    if args.sweep_only:
        # One plain elementwise kernel of known size ahead of the timed region (1 GiB read,
        # 1 GiB written): what a counter run of this command scales FETCH_SIZE and
        # WRITE_SIZE by.
        cal = torch.zeros(2, 1 << 28, dtype=torch.int32, device='cuda')
        torch.add(cal[0], 1, out=cal[1])
        torch.cuda.synchronize()
        del cal

    wall, us_launch = time_launches(lambda: prep.forward(x, route, y), args.steps,
                                    args.warmup, stream_ptr)
    kernel = _lib.load().sub1_last_kernel().decode()      # what the library launched
    assert prep.launch_faults(experts) == (0, 0)
    ms_per_step = wall / args.steps * 1e3
    abytes = algorithmic_bytes(stack, range(experts))
    achieved = abytes / (us_launch * 1e-6) / 1e9
    traffic, traffic_source = MEASURED_TRAFFIC.get(args.workload, (None, None)) \
        if not args.experts else (None, None)
    # what the kernel fetches: the entry stream once (the checkpoints behind it are not
    # read by the streaming kernel), row order and min/max of every slice, x and y
    fetched = int(prep.stream_bytes) + 6 * 64 * (-(-d_ff // 64) + -(-d_model // 64)) * experts \
        + 4 * experts * d_model

    out = {
        'metric': 'us per compressed MoE layer (batch-1) + achieved HBM GB/s vs roofline',
        'value': round(ms_per_step * 1e3, 2),
        'unit': 'us/layer',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'preheat_s': PREHEAT_S,       # untimed repeats of the step before the warm-up: clock ramp
        'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16 in/out, fp32 accumulate, u16 codes transcoded to 7-bit gap entries',
        'data': 'synthetic (seeded iid ternary experts, N(0,1) bf16 tokens)',
        'config': {'workload': desc, 'experts': experts, 'd_model': d_model, 'd_ff': d_ff,
                   'p_zero': p_zero, 'tokens': experts,
                   'compressed_bytes': stack.compressed_bytes(),
                   'bits_per_weight': round(16.0 * stack.w_comp.numel()
                                            / (2.0 * experts * d_model * d_ff), 4),
                   # the timed kernel reads a stream made ONCE from the codes, untimed:
                   'prepare_ms': round(prepare_ms, 1),
                   'prepared_stream_bytes': int(prep.stream_bytes),
                   'prepared_total_bytes': int(prep.code_bytes) + int(prep.meta.numel()),
                   'prepared_bits_per_weight': round(
                       8.0 * (int(prep.code_bytes) + int(prep.meta.numel()))
                       / (2.0 * experts * d_model * d_ff), 4),
                   # this process keeps the packed stack too (the other kernels and the CPU
                   # baseline read it); a layer needs the prepared pair alone to run
                   # (Sub1Experts.release_packed, checkpoint.load_prepared_experts)
                   'both_forms_resident': True,
                   'resident_bytes': {'packed': stack.compressed_bytes(),
                                      'prepared': int(prep.code_bytes) + int(prep.meta.numel()),
                                      'needed_to_run': int(prep.code_bytes) + int(prep.meta.numel())}},
        'roofline': {'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS,
                     'unit': 'GB/s', 'frac': round(achieved / HBM_PEAK_GBS, 4),
                     'traffic': traffic, 'traffic_source': traffic_source,
                     'kernel': kernel,
                     'algorithmic_bytes': abytes, 'us_per_launch': round(us_launch, 2),
                     # h (bf16 [d_ff] per token) is written by wi and read by wo in the
                     # algorithmic count; the fused kernel keeps it in LDS and moves neither
                     'algorithmic_bytes_excluding_h': abytes - 4 * d_ff * experts,
                     # codes, row offsets and min/max alone: the compressed bytes proper
                     'frac_on_compressed_bytes': round(
                         stack.compressed_bytes() / (us_launch * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     'fetched_bytes_by_layout': fetched,
                     'frac_on_fetched_bytes': round(
                         (traffic or fetched) / (us_launch * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)},
    }

    if args.sweep_only:
        print(json.dumps(out))
        return
    also = {}
    # batch-1: one token routed to one seeded uniform expert (launch-latency bound)
    g = torch.Generator().manual_seed(args.seed + 2)
    one = torch.randint(0, experts, (1,), generator=g).to(torch.int32).cuda()
    y1 = torch.empty_like(x[:1])
    _, us1 = time_launches(lambda: prep.forward(x[:1], one, y1), 200, 20, stream_ptr)
    also['single_token_us'] = round(us1, 2)
    # the same sweep through the kernel that reads the reference's packed layout directly
    y2 = torch.empty_like(x)
    _, us_ref = time_launches(lambda: stack.forward(x, route, y2), 3, 1, stream_ptr)
    also['reference_layout_kernel_us'] = round(us_ref, 1)
    # the same workload with the dictionary decoded inside the kernel, no preparation
    out['roofline']['reference_layout'] = {
        'kernel': _lib.load().sub1_last_kernel().decode(), 'us_per_launch': round(us_ref, 1),
        'frac': round(abytes / (us_ref * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)}
    also['prepared_vs_reference_layout_rel_diff'] = rel_diff(y, y2)
    if not also['prepared_vs_reference_layout_rel_diff'] <= 1e-2:
        raise SystemExit('the prepared kernel and the packed-layout kernel disagree on the sweep')
    # batched decode: 64 tokens routed top-1 by a seeded softmax router (skewed counts)
    t5 = 64
    x5 = synthetic.activations(t5, d_model, args.seed + 3)
    r5 = synthetic.softmax_router(t5, experts, args.seed + 4)
    y5 = torch.empty_like(x5)
    _, us5 = time_launches(lambda: prep.forward(x5, r5, y5), 100, 10, stream_ptr)
    y5b = stack.forward(x5, r5)
    also['routed_64_tokens'] = {'us_per_layer': round(us5, 2),
                                'experts_hit': int(torch.unique(r5).numel()),
                                'vs_reference_layout_kernel_rel_diff': rel_diff(y5, y5b)}
    # the batches in between, routed the same way
    also['routed_tokens_us'] = {}
    for t in (2, 4, 16, 32):
        xt = synthetic.activations(t, d_model, args.seed + 3)
        rt = synthetic.softmax_router(t, experts, args.seed + 4)
        yt = torch.empty_like(xt)
        _, us_t = time_launches(lambda: prep.forward(xt, rt, yt), 200, 20, stream_ptr)
        also['routed_tokens_us'][str(t)] = round(us_t, 2)
    if not args.no_dense:
        n = min(experts, 128)
        d_us = dense_gemv_us(stack, x, n)
        dense_bytes = experts * (4 * d_model * d_ff + 6 * d_model + 4 * d_ff)
        also['dense_bf16_gemv'] = {'us_per_expert_ffn': round(d_us, 2), 'experts_timed': n,
                                   'us_per_layer_extrapolated': round(d_us * experts, 1),
                                   'sub1_us_per_expert_ffn': round(us_launch / experts, 2),
                                   # torch.bmm runs far below the HBM rate on these shapes; the
                                   # bound a dense kernel cannot beat is its bytes at 8 TB/s
                                   'dense_bytes': dense_bytes,
                                   'us_per_layer_at_hbm_peak': round(dense_bytes / HBM_PEAK_GBS / 1e3, 1)}
    if not args.experts and args.workload == 'c2048-sweep':
        # the two smaller layers of the configuration list; their compressed stacks
        # (57 MB, 110 MB) fit the 256 MB last-level cache, so these are not HBM rates
        for name in ('base128', 'large128'):
            shp, n_e, p_z, _ = WORKLOADS[name]
            dm, df = synthetic.SHAPES[shp]
            st = synthetic.build_stack(n_e, dm, df, p_z, args.seed + 10)
            pr = st.prepare()
            xs = synthetic.activations(n_e, dm, args.seed + 11)
            rt = torch.arange(n_e, dtype=torch.int32, device='cuda')
            ys = torch.empty_like(xs)
            _, us_s = time_launches(lambda: pr.forward(xs, rt, ys), 100, 10, stream_ptr)
            ab = algorithmic_bytes(st, range(n_e))
            entry = {'us_per_layer': round(us_s, 2), 'algorithmic_bytes': ab,
                     'GBps_cache_resident': round(ab / us_s / 1e3, 1)}
            # batch 1 on this shape: one token to one expert, and two tokens to two
            for n_tok in (1, 2):
                y_few = torch.empty_like(xs[:n_tok])
                r_few = rt[5:5 + n_tok].contiguous()
                _, us_few = time_launches(lambda: pr.forward(xs[:n_tok], r_few, y_few), 500, 50,
                                          stream_ptr)
                entry['single_token_us' if n_tok == 1 else 'two_tokens_us'] = round(us_few, 2)
            if name == 'large128' and not args.no_dense:
                entry['dense_bf16_gemv_us_per_layer'] = round(dense_gemv_us(st, xs, n_e) * n_e, 1)
            entry.update(hbm_rate_by_rotation(name, args.seed + 40, stream_ptr))
            if not args.no_cpu:
                entry['cpu'] = cpu_layer_baseline(st, xs, min(16, len(os.sched_getaffinity(0))))
            if name == 'base128':
                # a large batch: 4096 tokens routed uniformly (32 per expert on
                # average), grouped by expert on the GPU, four tokens per walk
                gb = torch.Generator().manual_seed(args.seed + 12)
                xb = synthetic.activations(4096, dm, args.seed + 13)
                rb = torch.randint(0, n_e, (4096,), generator=gb).to(torch.int32).cuda()
                yb = torch.empty_like(xb)
                _, us_b = time_launches(lambda: pr.forward(xb, rb, yb), 30, 5, stream_ptr)
                entry['tokens4096_us_per_layer'] = round(us_b, 1)
                entry['faster_mlp'] = faster_mlp_protocol(st, args.seed + 14, stream_ptr)
            also[name] = entry
            del st, pr
    if not args.no_dense:
        also['single_matrix_1_token'] = single_matrix_protocol(args.seed + 30, stream_ptr)
    if not args.experts and args.workload == 'c2048-sweep':
        also['other_weight_statistics'] = density_sweep(args.seed + 50, stream_ptr)
    out['also'] = also

    if not args.no_cpu:
        available = len(os.sched_getaffinity(0))
        cores = min(16, available)          # threads used; a one-GPU box's share is 16
        done1, spent1 = cpu_baseline(stack, x, min(experts, 64), 1, budget_s=3.0)
        done, spent = cpu_baseline(stack, x, experts, cores)
        out['cpu_baseline'] = {
            'value': round(spent / done * experts * 1e6, 1), 'unit': 'us/layer', 'cores': cores,
            'cores_available': available,
            'kind': 'port',
            'sample': '%d of %d expert FFNs of the same stack through the scalar C oracle in '
                      'the reference kernel\'s lane order, %d at a time on %d host threads, '
                      '%.1f s, extrapolated to the layer' % (done, experts, cores, cores, spent),
            'one_core_us_per_layer': round(spent1 / done1 * experts * 1e6, 1),
            'one_core_sample': '%d expert FFNs, %.1f s' % (done1, spent1),
            'base_wi_3072x768_one_core_us': round(cpu_single_matrix_us(args.seed + 20), 1),
            'base_wi_3072x768_python_decode_matmul_us': round(cpu_python_decode_matmul_us(args.seed + 20), 1)}
    print(json.dumps(out))


if __name__ == '__main__':
    main()
