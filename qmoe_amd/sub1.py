"""Module surface of the reference's `sub1.py` for the compressed-layer path:
`setup`, the tables `dec`/`trie`, `GPUS`/`DEV`/`DEC`/`TRIE`, `Sub1Linear`
(same buffers, `forward(x)`, static `make(w)`), plus `Sub1Experts`, the
one-launch form of the expert loop, and `FasterMLP`, the sparse-MLP module the
reference wraps around it (router, expert launch, router-probability scaling).

Differences from the reference that a caller can observe:
  * importing works without a GPU (the reference indexes GPUS[-1] at import,
    sub1.py:107-111); the device tables are then empty until a GPU exists;
  * `Sub1Linear.forward` runs all tokens in one launch (the reference loops
    over tokens, sub1.py:137-142), from a gap-coded stream of the non-zero
    weights that it decodes from the codes on first use (`Sub1Linear.fast`);
  * any (height, width) works, not only the six Switch shapes.
"""
import torch
import torch.nn as nn

from . import sub1_hip


def setup():
    """(dec int32 [131072], trie int32 [65537, 9]) CPU tensors: the fixed
    dictionary, byte-identical to what reference sub1.py:29-102 builds."""
    return sub1_hip.build_tables()


dec, trie = setup()

# reference sub1.py:107-111; the last GPU is the default one there
GPUS = [torch.device('cuda:%d' % i) for i in range(torch.cuda.device_count())] \
    if torch.cuda.is_available() else []
DEV = GPUS[-1] if GPUS else None
DEC = [dec.to(gpu) for gpu in GPUS]
TRIE = trie.to(DEV) if DEV is not None else None


def device_tables(device):
    """(DEC for that device, TRIE moved to that device)."""
    device = torch.device(device)
    if device.type != 'cuda' or not GPUS:
        raise RuntimeError('the compressed-expert kernels need a GPU; got %s' % device)
    idx = device.index if device.index is not None else torch.cuda.current_device()
    t = TRIE if TRIE.device.index == idx else TRIE.to(device)
    return DEC[idx], t


class Sub1Linear(nn.Module):
    """Compressed linear layer (reference sub1.py:114-166): buffers `w_comp`
    int16 [comp_size], `row_off` int32 [height+1], `ter_minmax` bf16
    [2*height], and an empty bf16 `weight` that HuggingFace's Switch expert
    reads the dtype of."""

    def __init__(self, height, comp_size):
        super().__init__()
        self.register_buffer('w_comp', torch.zeros(comp_size, dtype=torch.int16))
        self.register_buffer('row_off', torch.zeros(height + 1, dtype=torch.int32))
        self.register_buffer('ter_minmax', torch.zeros(2 * height, dtype=torch.bfloat16))
        self.register_buffer('weight', torch.zeros(0, dtype=torch.bfloat16))

    # forward() goes through copies of the weights made from the codes on first
    # use (remade when a buffer is replaced or written in place): up to
    # `tile_tokens` - 1 tokens the prepared stream of the non-zero weights,
    # walked per token (about 1.1 times the bytes of w_comp: 0.78 against 0.69
    # bit per weight at 10% non-zeros), so that a token gets the same bits
    # whatever the number of tokens it comes with, as in the reference; from
    # `tile_tokens` tokens on the tile form that the matrix cores multiply from
    # (2 bits per weight whatever the density, about 2.9 times w_comp; results
    # equal to rounding, not to the bit; `tile_tokens = None` keeps long
    # sequences on the prepared stream and the tile copy unmade).
    # `packed_tokens = 2` sends one or two tokens straight through the packed
    # buffers instead, a wavefront per row: nothing is faster for a single
    # product (3.8 to 7.8 us of kernel time on the Switch shapes against 6.3 to
    # 8.4) and nothing is copied for it, but that kernel adds a row's terms in
    # another order, so a token's last bit then depends on the size of its batch.
    # `fast = False` runs from the packed buffers whatever the number of tokens.
    fast = True
    packed_tokens = 0
    tile_tokens = 64

    def _copy(self, kind, width):
        live = (self.w_comp, self.row_off, self.ter_minmax)
        key = tuple((t.data_ptr(), t._version, t.numel()) for t in live) + (width,)
        cache = self.__dict__.setdefault('_copies', {})
        cached = cache.get(kind)
        if cached is None or cached[0] != key:
            table = DEC[self.w_comp.device.index]
            make = sub1_hip.PreparedMatrix if kind == 'prepared' else sub1_hip.TiledMatrix
            # the entry keeps the source tensors alive: their addresses are part
            # of the key and must not be handed out again while it is cached
            cached = (key, make(table, self.w_comp, self.row_off, self.ter_minmax, width),
                      [t.detach() for t in live])
            cache[kind] = cached
        return cached[1]

    def _prepared(self, width):
        return self._copy('prepared', width)

    def forward(self, x):
        """x bf16 [T, width] -> bf16 [T, height] (reference sub1.py:132-143)."""
        height = self.row_off.shape[0] - 1
        y = torch.zeros((x.shape[0], height), dtype=torch.bfloat16, device=x.device)
        if x.shape[0] == 0:
            return y
        x = x.contiguous()
        if self.fast and self.tile_tokens is not None and x.shape[0] >= self.tile_tokens:
            self._copy('tiles', x.shape[1]).matvec_tokens(x, y)
        elif (self.fast and x.shape[0] > self.packed_tokens
              and x.shape[1] <= sub1_hip.PREPARED_MAX_WIDTH):
            self._prepared(x.shape[1]).matvec_tokens(x, y)
        else:
            table = DEC[self.w_comp.device.index]
            sub1_hip.sub1matvec_tokens(table, self.w_comp, self.row_off, self.ter_minmax, x, y)
        return y

    @staticmethod
    def make(w):
        """Ternarise and pack a dense matrix whose rows take the values
        {row min, 0, row max} (reference sub1.py:145-166; ties go to max)."""
        w = w.bfloat16()
        ter_minmax = torch.column_stack((w.min(1)[0], w.max(1)[0])).flatten()
        row_off = torch.zeros(w.shape[0] + 1, dtype=torch.int32, device=w.device)
        w_tern = torch.zeros(w.shape, dtype=torch.int32, device=w.device)
        w_tern[w == ter_minmax[0::2].reshape((-1, 1))] = 1
        w_tern[w == ter_minmax[1::2].reshape((-1, 1))] = 2
        _, table = device_tables(w.device)
        w_comp = sub1_hip.sub1pack(table, w_tern, row_off)

        linear = Sub1Linear(w.shape[0], w_comp.shape[0])
        linear.w_comp.data = w_comp
        linear.row_off.data = row_off
        linear.ter_minmax = ter_minmax
        return linear


class Sub1Experts(nn.Module):
    """All experts of one MoE layer behind one launch.

    Built from per-expert (wi, wo) `Sub1Linear` pairs; `forward(x, expert)`
    returns wo_e(relu(wi_e(x[t]))) per token and passes through tokens whose
    expert index is negative, which is what the loop at reference
    sub1.py:312-317 produces for routed and for dropped tokens."""

    def __init__(self, wi_layers, wo_layers):
        super().__init__()
        dev = wi_layers[0].w_comp.device
        self._dec = DEC[dev.index]
        # the layers' own tensors: read when a launcher is made, never copied whole
        self._wi = [(l.w_comp, l.row_off, l.ter_minmax) for l in wi_layers]
        self._wo = [(l.w_comp, l.row_off, l.ter_minmax) for l in wo_layers]
        self._d_ff = self._wi[0][1].numel() - 1
        self._d_model = self._wo[0][1].numel() - 1
        self._prepared = None
        self._stack = None

    # forward() goes through the prepared stream of the experts' non-zero
    # weights, made on first use straight from the layers' tensors (about 1.1
    # times their bytes; nothing else is allocated); set to False to run from the
    # packed buffers, through a stacked copy of them made on first use.  The
    # tensors are taken as fixed: after writing to them call refresh().
    fast = True

    @property
    def stack(self):
        """The experts' packed buffers back to back (an ExpertStack, a copy made
        on first use): what the launch that needs no preparation reads."""
        if self._wi is None:
            return None
        if self._stack is None:
            self._stack = sub1_hip.ExpertStack.from_layers(self._dec, self._wi, self._wo)
        return self._stack

    def can_prepare(self):
        return max(self._d_model, self._d_ff) <= sub1_hip.PREPARED_MAX_WIDTH

    def refresh(self):
        if self._wi is None:
            raise RuntimeError('the packed buffers were released; build the layer again')
        self._prepared = None
        self._stack = None

    def release_packed(self):
        """Keep only the prepared stream: makes it if need be and drops this
        module's references to the packed tensors and any stacked copy of them
        (the per-expert tensors the layer was built from are the caller's to
        drop).  What is lost is the way back: no refresh(), no run from the
        packed buffers.  A c-2048 model's 30 layers are ~135 GB packed and ~150 GB
        prepared: one 288 GB GPU holds one of the two."""
        if not self.can_prepare():
            raise RuntimeError('these shapes have no prepared form; the packed buffers stay')
        self.fast = True
        self._launcher()
        self._wi = self._wo = self._stack = None

    def _launcher(self):
        if self._wi is None:
            return self._prepared
        if not (self.fast and self.can_prepare()):
            return self.stack
        if self._prepared is None:
            self._prepared = sub1_hip.PreparedStack.from_layers(self._dec, self._wi, self._wo)
        return self._prepared

    def forward(self, x, expert_index):
        return self._launcher().forward(x.contiguous(),
                                        expert_index.to(torch.int32).contiguous())


def _router_outputs(outputs, experts):
    """(one-hot routing mask [.., E], top-1 probabilities [.., 1], the third
    output) from a Switch top-1 router's 3-tuple, in whichever form the
    installed transformers returns it:

      4.28 (reference sub1.py:310)  (mask [.., E] int, probs [.., 1], logits [.., E])
      5.x                           (probs [.., 1], mask [.., 1, E] int64, max prob [.., 1])

    The mask is the one integer tensor; a singleton top-k axis in front of its
    expert axis is squeezed.  Of the two floating tensors the probabilities are
    the one whose last dimension is 1; where both are (5.x, or a single
    expert), the one that comes first in the tuple."""
    outputs = tuple(outputs)
    if len(outputs) != 3:
        raise ValueError('a Switch top-1 router returns three tensors, got %d' % len(outputs))
    masks = [o for o in outputs if not o.is_floating_point()]
    floats = [o for o in outputs if o.is_floating_point()]
    if len(masks) != 1 or len(floats) != 2 or masks[0].shape[-1] != experts:
        raise ValueError('cannot tell the router outputs apart: %s'
                         % [(tuple(o.shape), o.dtype) for o in outputs])
    mask = masks[0]
    narrow = [o for o in floats if o.shape[-1] == 1]
    if not narrow:
        raise ValueError('no [.., 1] probabilities among the router outputs: %s'
                         % [tuple(o.shape) for o in outputs])
    probs = narrow[0]
    other = floats[1] if floats[0] is probs else floats[0]
    if mask.dim() == probs.dim() + 1 and mask.shape[-2] == 1:
        mask = mask.squeeze(-2)
    if mask.shape[:-1] != probs.shape[:-1]:
        raise ValueError('router mask %s and probabilities %s do not describe the same tokens'
                         % (tuple(mask.shape), tuple(probs.shape)))
    return mask, probs, other


class FasterMLP(nn.Module):
    """The sparse MLP of a Switch block around the compressed experts
    (reference sub1.py:299-321): router, experts, multiplication by the router
    probability.  `mlp` is the block's `SwitchTransformersSparseMLP`-shaped
    module: `mlp.router` and `mlp.experts` (a ModuleDict of modules with
    `wi`/`wo` Sub1Linear layers).

    Differences from the reference: the experts run in one launch, from a
    stacked copy of the layers' buffers made on first use (remade after .to(),
    load_state_dict or `refresh()`; the per-call check looks at four of the
    experts' tensors only, so other writes to the buffers need `refresh()`);
    tokens stay on their GPU (one GPU here, the reference moves them to the
    layer's GPU and back, sub1.py:307-320).

    `router_outputs`: what forward() returns.  True: the reference's pair
    `(hidden_states, (router_logits, expert_index))`, which the Switch block of
    transformers 4.28 unpacks; False: `hidden_states` alone, which the block of
    transformers 5.x adds to its residual.  None (default) follows the wrapped
    module: a sparse MLP whose forward is annotated to return a tensor gets the
    tensor, anything else the reference's pair."""

    def __init__(self, mlp, gpu=None, router_outputs=None):
        super().__init__()
        if gpu is not None:
            mlp = mlp.to(gpu)
        self.router = mlp.router
        self.experts = nn.ModuleList(mlp.experts.values())
        self.gpu = gpu
        if router_outputs is None:
            returns = getattr(getattr(type(mlp), 'forward', None), '__annotations__', {}).get('return')
            router_outputs = returns not in (torch.Tensor, 'torch.Tensor')
        self.router_outputs = bool(router_outputs)
        # the launch applies ReLU between wi and wo, as Switch's experts do
        # (HuggingFace's DenseActDense keeps its activation in `act`)
        for expert in self.experts:
            act = getattr(expert, 'act', None)
            if act is not None and not isinstance(act, nn.ReLU):
                raise ValueError('FasterMLP runs ReLU experts; this one has %r' % (act,))

    def _sentinels(self):
        # a few of the experts' tensors stand for all of them in the per-call
        # check (looking at every tensor of 2048 experts costs milliseconds)
        first, last = self.experts[0], self.experts[len(self.experts) - 1]
        return [first.wi.w_comp, first.wi.ter_minmax, last.wo.w_comp, last.wo.ter_minmax]

    def refresh(self):
        """Forget the stacked copy of the experts; the next forward rebuilds it.
        Call it after writing to or replacing expert buffers (moving the module
        with .to()/.cuda() and load_state_dict do it themselves)."""
        self._forget()

    def release_packed(self):
        """Keep only the prepared stream of this layer's experts: builds it if
        need be, then empties the experts' `w_comp`, `row_off` and `ter_minmax`
        buffers, which frees about half of the layer's memory.  From then on
        the layer can run and nothing else: saving it stores empty buffers, and
        moving, loading or refresh() raise."""
        launcher = self._launcher()
        if not isinstance(launcher, sub1_hip.PreparedStack):
            raise RuntimeError('these shapes have no prepared form; the packed buffers stay')
        self._released = True
        self._launcher_cache = (None, launcher, [])     # no aliases of expert tensors
        for expert in self.experts:
            for layer in (expert.wi, expert.wo):
                for name in ('w_comp', 'row_off', 'ter_minmax'):
                    old = getattr(layer, name)
                    setattr(layer, name, torch.zeros(0, dtype=old.dtype, device=old.device))
                layer.__dict__.pop("_copies", None)

    def _forget(self):
        if getattr(self, '_released', False):
            raise RuntimeError('the packed buffers of this layer were released; '
                               'it cannot be moved, reloaded or refreshed')
        self._launcher_cache = None

    def _apply(self, fn, *args, **kwargs):
        self._forget()
        return super()._apply(fn, *args, **kwargs)

    def _load_from_state_dict(self, *args, **kwargs):
        self._forget()
        return super()._load_from_state_dict(*args, **kwargs)

    def _launcher(self):
        cached = getattr(self, '_launcher_cache', None)
        if getattr(self, '_released', False):
            return cached[1]
        live = self._sentinels()
        key = tuple((t.data_ptr(), t._version, t.numel()) for t in live)
        if cached is None or cached[0] != key:
            layer = Sub1Experts([e.wi for e in self.experts], [e.wo for e in self.experts])
            # the aliases keep the keyed addresses from being reused while cached
            cached = (key, layer._launcher(), [t.detach() for t in live])
            self._launcher_cache = cached
        return cached[1]

    def forward(self, hidden_states):
        """hidden_states [B, S, d_model] -> router_probs * expert output (with
        `router_outputs` also (router_logits, expert_index), reference
        sub1.py:321); tokens that the router's capacity limit dropped keep
        their input (reference sub1.py:312-318)."""
        router_mask, router_probs, router_logits = _router_outputs(
            self.router(hidden_states), len(self.experts))
        # expert_index = argmax of the mask; a token the capacity limit dropped
        # has an all-zero mask row: expert -1 for the launch
        route, expert_index = sub1_hip.route_from_mask(router_mask)
        x = hidden_states.reshape(-1, hidden_states.shape[-1]).to(torch.bfloat16).contiguous()
        next_states = self._launcher().forward(x, route)
        hidden_states = router_probs * next_states.view(hidden_states.shape).to(hidden_states.dtype)
        if self.router_outputs:
            return hidden_states, (router_logits, expert_index)
        return hidden_states
