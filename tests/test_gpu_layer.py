"""The modules around the kernels: ternary front end -> make -> forward, and
the sparse-MLP module (router, one-launch experts, probability scaling) against
the reference's per-expert loop (sub1.py:306-321) restated with per-layer
calls."""
import os
import types

import pytest
import torch
import torch.nn as nn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def gpu():
    from qmoe_amd import sub1
    assert torch.cuda.is_available(), 'these tests need the GPU'
    assert sub1.DEC, 'device tables missing'
    return sub1


class Top1Router(nn.Module):
    """Switch top-1 router with a capacity limit, as HuggingFace's
    SwitchTransformersTop1Router computes it: fp32 softmax over a linear
    classifier, one-hot of the argmax, tokens beyond an expert's capacity (in
    sequence order) lose their expert.  `order` picks the tuple layout of
    transformers 4.28 ('mask_first') or of later versions ('probs_first')."""

    def __init__(self, d_model, experts, capacity, order):
        super().__init__()
        self.classifier = nn.Linear(d_model, experts, bias=False)
        self.experts, self.capacity, self.order = experts, capacity, order

    def forward(self, hidden):
        logits = self.classifier(hidden.float())
        probs = torch.softmax(logits, dim=-1)
        index = torch.argmax(probs, dim=-1)
        mask = torch.nn.functional.one_hot(index, self.experts)
        priority = torch.cumsum(mask, dim=-2)
        mask = mask * (priority <= self.capacity)
        top = torch.max(probs, dim=-1).values.unsqueeze(-1).to(hidden.dtype)
        if self.order == 'mask_first':
            return mask, top, logits
        return top, mask, logits


class Expert(nn.Module):
    def __init__(self, wi, wo):
        super().__init__()
        self.wi, self.wo = wi, wo

    def forward(self, x):
        return self.wo(torch.relu(self.wi(x)))


def ternary_dense(h, w, p0, gen):
    from qmoe_amd import synthetic
    t = synthetic.draw_symbols(h, w, p0, gen, 'cuda')
    mm = synthetic.draw_minmax(h, gen, 'cuda')
    lut = torch.stack((torch.zeros(h, device='cuda', dtype=torch.bfloat16), mm[0::2], mm[1::2]), 1)
    return torch.gather(lut, 1, t.long()).contiguous()


def test_ternarize_make_forward(gpu):
    from qmoe_amd import quant, sub1, sub1_hip
    g = torch.Generator(device='cuda').manual_seed(31)
    w = torch.randn((192, 320), generator=g, device='cuda') * 0.05
    wq = quant.ternarize(w)
    lin = sub1.Sub1Linear.make(wq)
    dense = sub1_hip.sub1decode(sub1.DEC[0], lin.w_comp, lin.row_off, lin.ter_minmax, 320,
                                want_tern=False)[1]
    assert torch.equal(dense, wq.bfloat16())          # the packed layer holds exactly wq
    x = torch.randn((5, 320), generator=g, device='cuda').bfloat16()
    y = lin(x)
    ref = x.float() @ wq.bfloat16().float().t()
    assert torch.linalg.norm(y.float() - ref) <= 1e-2 * torch.linalg.norm(ref)
    # compression: far below 2 bytes per weight
    assert lin.w_comp.numel() * 2 < 0.2 * w.numel() * 2


@pytest.mark.parametrize('dtype', [torch.int64, torch.int32, torch.uint8, torch.bool])
def test_route_from_mask_is_argmax_with_dropped_tokens(gpu, dtype):
    """token_expert from a router's mask in one launch: the argmax over the
    experts (reference sub1.py:311), -1 where a token's row is all zero
    (reference sub1.py:312-318); one-hot rows, all-zero rows, expert counts
    that are no multiple of the wavefront, and rows with several ones (the first
    wins, as in torch.argmax)."""
    from qmoe_amd import sub1_hip
    g = torch.Generator().manual_seed(5)
    for batch, seq, experts in ((2, 37, 128), (1, 1, 2048), (3, 5, 7), (1, 300, 1), (1, 9, 65)):
        pick = torch.randint(0, experts, (batch, seq), generator=g)
        mask = torch.nn.functional.one_hot(pick, experts)
        mask[0, 0] = 0                       # a dropped token
        if seq > 3:
            mask[-1, 3] = 0
            mask[-1, 2, experts // 2:] = 1   # several ones
        mask = mask.to(dtype).cuda()
        route, index = sub1_hip.route_from_mask(mask)
        want = torch.argmax(mask.to(torch.int64), dim=-1)
        assert index.dtype == torch.int64 and index.shape == mask.shape[:-1]
        assert torch.equal(index, want)
        dropped = ~mask.to(torch.bool).any(dim=-1)
        assert route.dtype == torch.int32 and route.shape == (batch * seq,)
        assert torch.equal(route, torch.where(dropped, -1, want).reshape(-1).to(torch.int32))
    if dtype == torch.int64:
        # a general integer mask: the first largest element, negative values are non-zero
        mask = torch.tensor([[0, 3, 3, 1], [-2, -1, -1, -5], [0, 0, 0, 0]], device='cuda')
        route, index = sub1_hip.route_from_mask(mask)
        assert index.tolist() == [1, 1, 0] and route.tolist() == [1, 1, -1]
    empty = torch.zeros((0, 8), dtype=dtype, device='cuda')
    route, index = sub1_hip.route_from_mask(empty)
    assert route.numel() == 0 and index.numel() == 0
    with pytest.raises(TypeError):
        sub1_hip.route_from_mask(torch.zeros((2, 4), device='cuda'))



@pytest.mark.parametrize('order', ['mask_first', 'probs_first'])
def test_faster_mlp_equals_the_expert_loop(gpu, order):
    from qmoe_amd import sub1
    d_model, d_ff, experts, batch, seq = 256, 512, 6, 2, 24
    g = torch.Generator(device='cuda').manual_seed(41)
    layers = nn.ModuleDict()
    for e in range(experts):
        wi = sub1.Sub1Linear.make(ternary_dense(d_ff, d_model, 0.85, g))
        wo = sub1.Sub1Linear.make(ternary_dense(d_model, d_ff, 0.85, g))
        layers['expert_%d' % e] = Expert(wi, wo)
    router = Top1Router(d_model, experts, capacity=3, order=order).cuda()
    with torch.no_grad():
        router.classifier.weight.copy_(torch.randn((experts, d_model), generator=g, device='cuda'))
    mlp = types.SimpleNamespace(router=router, experts=layers)
    fast = sub1.FasterMLP(mlp)
    hidden = torch.randn((batch, seq, d_model), generator=g, device='cuda').bfloat16()
    out, (logits, index) = fast(hidden)

    # the reference's loop, per expert (reference sub1.py:311-318)
    outs = router(hidden)
    mask, probs = (outs[0], outs[1]) if order == 'mask_first' else (outs[1], outs[0])
    assert int((mask.sum(-1) == 0).sum()) > 0            # the capacity limit dropped tokens

    def expert_loop():
        next_states = hidden.clone()
        for e in torch.nonzero(mask.sum(dim=(0, 1)), as_tuple=True)[0]:
            sel = mask[:, :, e].bool()
            next_states[sel] = layers['expert_%d' % int(e)](hidden[sel])
        return probs * next_states

    want = expert_loop()
    assert torch.equal(out, want)
    # and with the layers on their packed buffers, which add in another order
    saved = sub1.Sub1Linear.fast
    sub1.Sub1Linear.fast = False
    try:
        packed = expert_loop()
    finally:
        sub1.Sub1Linear.fast = saved
    assert torch.linalg.norm(out.float() - packed.float()) <= 1e-2 * torch.linalg.norm(packed.float())
    assert torch.equal(index, torch.argmax(mask, dim=-1))
    assert torch.equal(logits, outs[2])
    # a second call reuses the stacked experts
    stacked = fast._launcher()
    assert torch.equal(fast(hidden)[0], want)
    assert fast._launcher() is stacked
    # writing to an expert in the middle is seen after refresh(); moving the module remakes the copy too
    mid = layers['expert_2']
    mid.wo.ter_minmax.mul_(2)
    fast.refresh()
    assert fast._launcher() is not stacked
    assert torch.equal(fast(hidden)[0], expert_loop())
    stacked = fast._launcher()
    fast.cuda()
    assert fast._launcher() is not stacked


def test_faster_mlp_in_a_huggingface_sparse_mlp(gpu):
    """A SwitchTransformersSparseMLP of the installed transformers, built from
    a config (nothing is fetched), its experts' wi/wo replaced by
    Sub1Linear.make(...): FasterMLP around it equals the reference's loop
    (sub1.py:306-321) on the same modules bit for bit, returns what the
    installed Switch block expects from its mlp, and agrees with HuggingFace's
    own expert loop on the compressed experts to bf16 rounding."""
    pytest.importorskip('transformers')
    from transformers.models.switch_transformers import modeling_switch_transformers as hf
    from qmoe_amd import sub1
    d_model, d_ff, experts, batch, seq = 256, 512, 8, 2, 40
    cfg = hf.SwitchTransformersConfig(d_model=d_model, d_ff=d_ff, num_experts=experts,
                                      expert_capacity=64, num_layers=2,
                                      num_sparse_encoder_layers=1, num_heads=4, d_kv=64,
                                      vocab_size=128, router_jitter_noise=0.0, dropout_rate=0.0)
    torch.manual_seed(43)
    block = hf.SwitchTransformersLayerFF(cfg, is_sparse=True).cuda().bfloat16().eval()
    mlp = block.mlp
    assert isinstance(mlp, hf.SwitchTransformersSparseMLP)
    g = torch.Generator(device='cuda').manual_seed(44)
    for e in range(experts):
        expert = mlp.experts['expert_%d' % e]
        expert.wi = sub1.Sub1Linear.make(ternary_dense(d_ff, d_model, 0.85, g))
        expert.wo = sub1.Sub1Linear.make(ternary_dense(d_model, d_ff, 0.85, g))
    hidden = torch.randn((batch, seq, d_model), generator=g, device='cuda').bfloat16()
    fast = sub1.FasterMLP(mlp)
    with torch.no_grad():
        got = fast(hidden)
        router_mask, router_probs, _ = sub1._router_outputs(mlp.router(hidden), experts)
        # reference sub1.py:311-318 on the same modules
        next_states = hidden.clone()
        for e in torch.nonzero(router_mask.sum(dim=(0, 1)), as_tuple=True)[0]:
            sel = router_mask[:, :, e].bool()
            next_states[sel] = mlp.experts['expert_%d' % int(e)](hidden[sel])
        want = router_probs * next_states
        theirs = mlp(hidden)
    pair = isinstance(theirs, tuple)
    assert fast.router_outputs is pair
    if pair:
        got, theirs = got[0], theirs[0]
    assert len(torch.unique(router_mask.argmax(-1))) > 1      # several experts hit
    assert torch.equal(got, want)
    assert torch.linalg.norm(got.float() - theirs.float()) <= 1e-2 * torch.linalg.norm(theirs.float())
    # plugged into the block: layer norm, the compressed sparse MLP, residual
    with torch.no_grad():
        plain = block(hidden)
        block.mlp = fast
        plugged = block(hidden)
    plain = plain[0] if isinstance(plain, tuple) else plain
    plugged = plugged[0] if isinstance(plugged, tuple) else plugged
    assert torch.linalg.norm(plugged.float() - plain.float()) <= 1e-2 * torch.linalg.norm(plain.float())


def test_faster_mlp_refuses_other_activations(gpu):
    """The launch computes ReLU between the projections; an expert that says it
    uses another activation (HuggingFace keeps it in `act`) is refused."""
    sub1 = gpu
    g = torch.Generator(device='cuda').manual_seed(59)
    expert = Expert(sub1.Sub1Linear.make(ternary_dense(64, 32, 0.8, g)),
                    sub1.Sub1Linear.make(ternary_dense(32, 64, 0.8, g)))
    expert.act = nn.GELU()
    mlp = types.SimpleNamespace(router=Top1Router(32, 1, 4, 'probs_first').cuda(),
                                experts=nn.ModuleDict({'expert_0': expert}))
    with pytest.raises(ValueError, match='ReLU'):
        sub1.FasterMLP(mlp)
    expert.act = nn.ReLU()
    sub1.FasterMLP(mlp)


def test_checkpoint_directory_to_one_launch_layer(gpu, tmp_path):
    """Experts written in the reference's directory format come back as one
    stacked layer whose output equals the per-expert layers' output."""
    from qmoe_amd import checkpoint, sub1
    d_model, d_ff, experts = 128, 320, 4
    g = torch.Generator(device='cuda').manual_seed(51)
    mgr = checkpoint.Sub1CheckpointManager(str(tmp_path), config={'d_model': d_model})
    made = []
    for j in range(experts):
        wi = sub1.Sub1Linear.make(ternary_dense(d_ff, d_model, 0.8, g))
        wo = sub1.Sub1Linear.make(ternary_dense(d_model, d_ff, 0.8, g))
        made.append(Expert(wi, wo))
        mgr.add_expert('decoder.block.1.layer.2.mlp.experts.expert_%d' % j, wi, wo)
    mgr.finalize()
    stacks = checkpoint.load_expert_stacks(str(tmp_path), 'cuda:0')
    assert list(stacks) == ['decoder.block.1.layer.2.mlp']
    layer = stacks['decoder.block.1.layer.2.mlp']
    x = torch.randn((9, d_model), generator=g, device='cuda').bfloat16()
    route = torch.tensor([0, 3, 1, 2, 2, -1, 0, 3, 1], dtype=torch.int32, device='cuda')
    y = layer(x, route)
    for t in range(9):
        e = int(route[t])
        want = x[t:t + 1] if e < 0 else made[e](x[t:t + 1])
        assert torch.equal(y[t:t + 1], want), t


def test_checkpoint_directory_to_prepared_only_layers(gpu, tmp_path):
    """The loader for models too large to hold twice: two layers whose experts
    are spread over three files, out of order, come back as prepared-only
    layers that give the bits of the stacked layers and hold no packed copy."""
    from qmoe_amd import checkpoint, sub1, sub1_hip
    d_model, d_ff, experts = 128, 320, 4
    g = torch.Generator(device='cuda').manual_seed(53)
    mgr = checkpoint.Sub1CheckpointManager(str(tmp_path), config={'d_model': d_model})
    names = [('encoder.block.1.layer.1.mlp', j) for j in (3, 0, 2, 1)] + \
            [('decoder.block.1.layer.2.mlp', j) for j in (1, 0, 3, 2)]
    for n, (layer_name, j) in enumerate(names):
        wi = sub1.Sub1Linear.make(ternary_dense(d_ff, d_model, 0.8, g))
        wo = sub1.Sub1Linear.make(ternary_dense(d_model, d_ff, 0.8, g))
        mgr.add_expert('%s.experts.expert_%d' % (layer_name, j), wi, wo)
        if n in (2, 5):                      # files end in the middle of a layer
            mgr.save_experts()
    mgr.finalize()
    assert sorted(f for f in os.listdir(str(tmp_path)) if f.startswith('exp')) == \
        ['exp00.pt', 'exp01.pt', 'exp02.pt']
    stacks = checkpoint.load_expert_stacks(str(tmp_path), 'cuda:0')
    lean = checkpoint.load_prepared_experts(str(tmp_path), 'cuda:0')
    assert set(lean) == set(stacks) and len(lean) == 2
    x = torch.randn((9, d_model), generator=g, device='cuda').bfloat16()
    route = torch.tensor([0, 3, 1, 2, 2, -1, 0, 3, 1], dtype=torch.int32, device='cuda')
    for name, layer in lean.items():
        assert layer.stack is None and isinstance(layer._launcher(), sub1_hip.PreparedStack)
        assert torch.equal(layer(x, route), stacks[name](x, route)), name
        with pytest.raises(RuntimeError):
            layer.refresh()
    # a layer with an expert missing from the files
    os.remove(os.path.join(str(tmp_path), 'exp01.pt'))
    with pytest.raises(ValueError):
        checkpoint.load_prepared_experts(str(tmp_path), 'cuda:0')


def test_faster_mlp_release_packed(gpu):
    """release_packed() frees the experts' packed buffers (the memory in use
    drops by their size), the layer keeps giving the same bits, and what can
    no longer work raises."""
    sub1 = gpu
    d_model, d_ff, n = 256, 640, 16
    g = torch.Generator(device='cuda').manual_seed(57)
    experts = nn.ModuleDict()
    for j in range(n):
        experts['expert_%d' % j] = Expert(
            sub1.Sub1Linear.make(ternary_dense(d_ff, d_model, 0.85, g)),
            sub1.Sub1Linear.make(ternary_dense(d_model, d_ff, 0.85, g)))
    mlp = types.SimpleNamespace(router=Top1Router(d_model, n, 3, 'probs_first').cuda(),
                                experts=experts)
    fast = sub1.FasterMLP(mlp)
    hidden = torch.randn((2, 24, d_model), generator=g, device='cuda').bfloat16()
    want = fast(hidden)[0].clone()
    packed = sum(t.numel() * t.element_size() for e in fast.experts for l in (e.wi, e.wo)
                 for t in (l.w_comp, l.row_off, l.ter_minmax))
    del experts, mlp
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    fast.release_packed()
    torch.cuda.synchronize()
    freed = before - torch.cuda.memory_allocated()
    assert freed >= 0.9 * packed, (freed, packed)
    assert all(e.wi.w_comp.numel() == 0 and e.wo.ter_minmax.numel() == 0 for e in fast.experts)
    assert torch.equal(fast(hidden)[0], want)
    assert torch.equal(fast(hidden)[0], want)
    for broken in (fast.refresh, fast.cuda, lambda: fast.load_state_dict(fast.state_dict())):
        with pytest.raises(RuntimeError):
            broken()


def test_layer_launch_replays_from_a_graph(gpu):
    """The grouped launch allocates nothing and clears its control words with
    a kernel, so a HIP graph can hold it: replays (with eager launches and
    synchronisations in between) give the eager result every time."""
    from qmoe_amd import synthetic
    d_model, d_ff = synthetic.SHAPES['base']
    stack = synthetic.build_stack(8, d_model, d_ff, 0.9, seed=61)
    prep = stack.prepare()
    for tokens in (1, 12):
        x = synthetic.activations(tokens, d_model, seed=62)
        route = (torch.arange(tokens, dtype=torch.int32, device='cuda') * 3) % 8
        y = torch.empty_like(x)
        prep.forward(x, route, y)            # first call: workspace
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            prep.forward(x, route, y)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            prep.forward(x, route, y)
        for rep in range(4):
            x.copy_(synthetic.activations(tokens, d_model, seed=70 + rep))
            y.zero_()
            graph.replay()
            torch.cuda.synchronize()
            got = y.clone()
            eager = prep.forward(x, route)   # eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(got, eager), (tokens, rep)


def test_a_large_layer_is_prepared_without_a_second_packed_copy(gpu):
    """256 experts of the Switch-c-2048 shapes (0.58 GB packed): building the
    one-launch layer from the experts' own tensors and running it allocates the
    prepared pair and little else (no stacked copy of the packed buffers on the
    way), and with the packed tensors released the layer holds the prepared pair
    alone.  The stream is the one that preparing a stacked copy gives."""
    sub1 = gpu
    from qmoe_amd import sub1_hip, synthetic
    d_model, d_ff = synthetic.SHAPES['c2048']
    experts = 256
    torch.cuda.synchronize()
    before_stack = torch.cuda.memory_allocated()      # whatever earlier tests still hold
    stack = synthetic.build_stack(experts, d_model, d_ff, 0.9, seed=4242)
    packed = stack.compressed_bytes()
    triples = [synthetic.expert_layers(stack, e) for e in range(experts)]

    def as_layer(t):
        return types.SimpleNamespace(w_comp=t[0], row_off=t[1], ter_minmax=t[2])

    wi_layers = [as_layer(wi) for wi, _ in triples]
    wo_layers = [as_layer(wo) for _, wo in triples]
    x = synthetic.activations(48, d_model, seed=5)
    route = (torch.arange(48, dtype=torch.int32, device='cuda') * 5) % experts
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    layer = sub1.Sub1Experts(wi_layers, wo_layers)
    y = layer(x, route)
    torch.cuda.synchronize()
    prep = layer._launcher()
    assert isinstance(prep, sub1_hip.PreparedStack)
    prepared = prep.codes.numel() + prep.meta.numel()
    peak = torch.cuda.max_memory_allocated() - base
    assert peak <= 1.05 * prepared, (peak, prepared, packed)
    assert base + peak - before_stack <= 1.05 * (packed + prepared)
    # the same stream as from the stacked copy, and the same results
    other = stack.prepare()
    assert prep.meta.numel() == other.meta.numel()       # (the gaps between its arrays hold anything)
    assert torch.equal(prep.codes[:int(prep._c.total_chunks) * 512], other.codes[:int(other._c.total_chunks) * 512])
    assert torch.equal(y, other.forward(x, route))
    del other
    # one resident form: the prepared pair alone
    layer.release_packed()
    del stack, triples, wi_layers, wo_layers
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated() - before_stack
    small = x.numel() * 2 * 2 + route.numel() * 4 + sum(w.numel() for w in prep._ws.values())
    assert held <= 1.05 * prepared + small, (held, prepared)
    assert torch.equal(layer(x, route), y)
