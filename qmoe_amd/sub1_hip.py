"""Operator module with the surface of the reference's `sub1_cuda` extension
(reference sub1_cuda.cpp:56-59): `sub1matvec` and `sub1pack`, same positional
arguments, tensors in, launched on torch's current stream.  Underneath is the C
ABI of libsub1_hip.so; torch only supplies device memory and the stream.

    import qmoe_amd.sub1_hip as sub1_cuda      # drop-in for `import sub1_cuda`

Additions the reference does not have: argument checking (the reference casts
raw pointers unchecked and silently ignores unsupported shapes,
sub1_cuda_kernel.cu:78-87), `sub1matvec_tokens`, `sub1decode`, and the grouped
expert launch `ExpertStack.forward`.
"""
import ctypes

import torch

from . import _lib

DICT_ENTRIES = _lib.DICT_ENTRIES
PREPARED_MAX_WIDTH = _lib.PREPARED_MAX_WIDTH
Sub1Fault = _lib.Sub1Fault
check_faults = _lib.check_faults


def clear_faults():
    """Reset the library's fault flags once the work that raised them has
    ended (synchronise first).  The stacks zero their workspaces again before
    their next launch, and the static scratch of the launch that does not
    allocate is zeroed here, on the current stream."""
    _lib.clear_faults(_stream())


def _stream():
    """torch's current stream on the current device, as the C ABI takes it."""
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


class _on_device:
    """`with _on_device(dev):` makes dev the current device for the launch; a
    device that already is costs two cheap calls instead of torch's guard."""

    def __init__(self, device):
        self.want = device.index if device.index is not None else torch._C._cuda_getDevice()
        self.guard = None

    def __enter__(self):
        if torch._C._cuda_getDevice() != self.want:
            self.guard = torch.cuda.device(self.want)
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _need(t, dtype, name, device=None, numel=None, dim=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError('%s must be a torch.Tensor' % name)
    if t.dtype != dtype:
        raise TypeError('%s must be %s, got %s' % (name, dtype, t.dtype))
    if not t.is_cuda:
        raise ValueError('%s must live on the GPU' % name)
    if device is not None and t.device != device:
        raise ValueError('%s is on %s, expected %s' % (name, t.device, device))
    if not t.is_contiguous():
        raise ValueError('%s must be contiguous' % name)
    if numel is not None and t.numel() != numel:
        raise ValueError('%s must hold %d elements, got %d' % (name, numel, t.numel()))
    if dim is not None and t.dim() != dim:
        raise ValueError('%s must be %d-D' % (name, dim))
    return t.data_ptr()


def route_from_mask(router_mask):
    """(route int32 [T], expert_index int64 shaped like the mask without its
    last dimension) from a top-1 router's mask [..., E] in one launch:
    expert_index = argmax over the experts (reference sub1.py:311), route the
    same with -1 for a token whose row is all zero (dropped by the router's
    capacity limit: it keeps its input, reference sub1.py:312-318)."""
    if not isinstance(router_mask, torch.Tensor) or not router_mask.is_cuda:
        raise ValueError('router_mask must be a tensor on the GPU')
    size = {torch.int64: 8, torch.int32: 4, torch.uint8: 1, torch.bool: 1}.get(router_mask.dtype)
    if size is None:
        raise TypeError('router_mask must be int64, int32, uint8 or bool, got %s' % router_mask.dtype)
    mask = router_mask.contiguous()
    experts = mask.shape[-1]
    tokens = mask.numel() // experts if experts else 0
    route = torch.empty(tokens, dtype=torch.int32, device=mask.device)
    index = torch.empty(mask.shape[:-1], dtype=torch.int64, device=mask.device)
    if tokens == 0:
        return route, index
    with _on_device(mask.device):
        _lib.check(_lib.load().sub1_route_from_mask(mask.data_ptr(), size, tokens, experts,
                                                    route.data_ptr(), index.data_ptr(), _stream()))
    return route, index


def build_tables():
    """(dec int32 [131072], trie int32 [65537, 9]) on the CPU: the fixed
    dictionary of reference sub1.py:29-102, built by the library (C++)."""
    dec = torch.empty(_lib.DEC_WORDS, dtype=torch.int32)
    trie = torch.empty((_lib.TRIE_ROWS, 9), dtype=torch.int32)
    _lib.check(_lib.load().sub1_build_tables(dec.data_ptr(), trie.data_ptr()))
    return dec, trie


def sub1matvec(dec, w_comp, row_off, ter_minmax, x, y):
    """y += W x for one compressed matrix; height = y.numel(), width =
    x.numel() (reference sub1_cuda_kernel.cu:78-79).  Any shape, in place."""
    dev = dec.device if isinstance(dec, torch.Tensor) else None
    _lib.check_faults()
    height, width = y.numel(), x.numel()
    args = [
        _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS),
        _need(w_comp, torch.int16, 'w_comp', dev),
        _need(row_off, torch.int32, 'row_off', dev, numel=height + 1),
        _need(ter_minmax, torch.bfloat16, 'ter_minmax', dev, numel=2 * height),
        _need(x, torch.bfloat16, 'x', dev),
        _need(y, torch.bfloat16, 'y', dev),
    ]
    with _on_device(dev):
        _lib.check(_lib.load().sub1_matvec(*args, height, width, _stream()))


def sub1matvec_tokens(dec, w_comp, row_off, ter_minmax, x, y):
    """y[t] += W x[t] for x [T, W], y [T, H] in one launch."""
    dev = dec.device if isinstance(dec, torch.Tensor) else None
    args = [
        _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS),
        _need(w_comp, torch.int16, 'w_comp', dev),
        _need(row_off, torch.int32, 'row_off', dev),
        _need(ter_minmax, torch.bfloat16, 'ter_minmax', dev),
        _need(x, torch.bfloat16, 'x', dev, dim=2),
        _need(y, torch.bfloat16, 'y', dev, dim=2),
    ]
    tokens, width = x.shape
    height = row_off.numel() - 1
    if y.shape != (tokens, height) or ter_minmax.numel() != 2 * height:
        raise ValueError('y must be [%d, %d] and ter_minmax [%d]' % (tokens, height, 2 * height))
    with _on_device(dev):
        _lib.check(_lib.load().sub1_matvec_tokens(*args, height, width, tokens,
                                                  width, height, _stream()))


def sub1pack(trie, w_tern, row_off):
    """Greedy dictionary encode of w_tern (int32 [H, W] symbols, CLOBBERED);
    row_off (int32 [H+1]) is overwritten with the cumulative code counts and
    the int16 code stream is returned (reference sub1_cuda_kernel.cu:92-126)."""
    dev = trie.device if isinstance(trie, torch.Tensor) else None
    p_trie = _need(trie, torch.int32, 'trie', numel=_lib.TRIE_ROWS * 9)
    p_w = _need(w_tern, torch.int32, 'w_tern', dev, dim=2)
    height, width = w_tern.shape
    p_ro = _need(row_off, torch.int32, 'row_off', dev, numel=height + 1)
    lib = _lib.load()
    with _on_device(dev):
        _lib.check(lib.sub1_pack_count(p_trie, p_w, p_ro, height, width, _stream()))
        total = int(row_off[height].item())      # the one host sync, as in the reference
        w_comp = torch.empty(total, dtype=torch.int16, device=dev)
        _lib.check(lib.sub1_pack_emit(p_w, p_ro, w_comp.data_ptr(), height, width, _stream()))
    return w_comp


def sub1decode(dec, w_comp, row_off, ter_minmax, width, want_tern=True, want_w=True):
    """Decode without multiplying: (symbols uint8 [H, W] or None, weights bf16
    [H, W] or None, number of rows whose codes do not cover the width)."""
    dev = dec.device if isinstance(dec, torch.Tensor) else None
    height = row_off.numel() - 1
    p_dec = _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS)
    p_wc = _need(w_comp, torch.int16, 'w_comp', dev)
    p_ro = _need(row_off, torch.int32, 'row_off', dev)
    p_mm = _need(ter_minmax, torch.bfloat16, 'ter_minmax', dev, numel=2 * height) \
        if ter_minmax is not None else None
    tern = torch.zeros((height, width), dtype=torch.uint8, device=dev) if want_tern else None
    w = torch.zeros((height, width), dtype=torch.bfloat16, device=dev) if want_w else None
    bad = torch.zeros(1, dtype=torch.int32, device=dev)
    with _on_device(dev):
        _lib.check(_lib.load().sub1_decode(
            p_dec, p_wc, p_ro, p_mm, tern.data_ptr() if want_tern else None,
            w.data_ptr() if want_w else None, bad.data_ptr(), height, width, _stream()))
    return tern, w, int(bad.item())


def _workspace(stack, tokens):
    """The launch's scratch memory (control words and h), one buffer per
    stream: launches on different streams may run at once, launches on one
    stream run in order and share theirs.  Zeroed when it is made; the
    launches leave its control words at zero again, except that a wait which
    gave up may not: once such a fault has been cleared (clear_faults moves
    fault_epoch on), every buffer made before that is zeroed again at its next
    use.  A buffer that has to grow is replaced; the old one goes back to
    torch's allocator, which hands it out again only in the order of the stream
    it was allocated on."""
    need = _lib.load().sub1_moe_workspace_bytes(tokens, stack.d_ff)
    key = _stream().value
    epoch = _lib.fault_epoch()
    ws = stack._ws.get(key)
    if ws is None or ws.numel() < need:
        with _on_device(stack.device):
            ws = torch.zeros(need, dtype=torch.uint8, device=stack.device)
        stack._ws[key] = ws
        stack._seen[key] = (0, 0)
        stack._ws_epoch[key] = epoch
    elif stack._ws_epoch.get(key) != epoch:
        ws.zero_()
        stack._seen[key] = (0, 0)
        stack._ws_epoch[key] = epoch
    return ws


def _fault_delta(stack, tokens):
    # words 1 and 2 of the workspace count over all launches; report what is new
    key = _stream().value
    ctrl = stack.workspace(tokens)[:16].view(torch.int32).tolist()
    before = stack._seen.get(key, (0, 0))
    stack._seen[key] = (ctrl[1], ctrl[2])
    return (ctrl[1] - before[0]) & 0xffffffff, (ctrl[2] - before[1]) & 0xffffffff


class ExpertStack:
    """The Sub1Linear buffers of all experts of one MoE layer, back to back in
    one set of tensors, and the one-launch forward over them.

    wi[e], wo[e] are (w_comp int16 [C], row_off int32 [H+1], ter_minmax bf16
    [2H]) triples as Sub1Linear holds them; wi has H = d_ff, wo has H = d_model.
    """

    def __init__(self, dec, w_comp, wi_code_base, wo_code_base, wi_row_off, wo_row_off,
                 wi_minmax, wo_minmax, d_model, d_ff):
        dev = dec.device
        experts = wi_code_base.numel()
        self.dec, self.w_comp = dec, w_comp
        self.wi_code_base, self.wo_code_base = wi_code_base, wo_code_base
        self.wi_row_off, self.wo_row_off = wi_row_off, wo_row_off
        self.wi_minmax, self.wo_minmax = wi_minmax, wo_minmax
        self.experts, self.d_model, self.d_ff = experts, d_model, d_ff
        self.device = dev
        self._c = _lib.MoeStack(
            _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS),
            _need(w_comp, torch.int16, 'w_comp', dev),
            _need(wi_code_base, torch.int64, 'wi_code_base', dev, numel=experts),
            _need(wo_code_base, torch.int64, 'wo_code_base', dev, numel=experts),
            _need(wi_row_off, torch.int32, 'wi_row_off', dev, numel=experts * (d_ff + 1)),
            _need(wo_row_off, torch.int32, 'wo_row_off', dev, numel=experts * (d_model + 1)),
            _need(wi_minmax, torch.bfloat16, 'wi_minmax', dev, numel=experts * 2 * d_ff),
            _need(wo_minmax, torch.bfloat16, 'wo_minmax', dev, numel=experts * 2 * d_model),
            experts, d_model, d_ff)
        self._ws = {}
        self._ws_epoch = {}  # per workspace: fault_epoch() when it was last zeroed
        self._seen = {}      # per workspace: the fault counts launch_faults() last returned from

    @classmethod
    def from_layers(cls, dec, wi_layers, wo_layers):
        """Stack per-expert (w_comp, row_off, ter_minmax) triples."""
        dev = dec.device
        d_ff = wi_layers[0][1].numel() - 1
        d_model = wo_layers[0][1].numel() - 1
        sizes = [t[0].numel() for t in wi_layers] + [t[0].numel() for t in wo_layers]
        bases = torch.zeros(len(sizes) + 1, dtype=torch.int64)
        bases[1:] = torch.tensor(sizes, dtype=torch.int64).cumsum(0)
        n = len(wi_layers)
        w_comp = torch.cat([t[0] for t in wi_layers] + [t[0] for t in wo_layers])
        return cls(dec, w_comp, bases[:n].to(dev), bases[n:2 * n].to(dev),
                   torch.cat([t[1] for t in wi_layers]), torch.cat([t[1] for t in wo_layers]),
                   torch.cat([t[2] for t in wi_layers]), torch.cat([t[2] for t in wo_layers]),
                   d_model, d_ff)

    def compressed_bytes(self):
        """Bytes of the stack a full sweep reads: codes, row offsets, min/max."""
        return (2 * self.w_comp.numel() + 4 * self.wi_row_off.numel()
                + 4 * self.wo_row_off.numel() + 2 * self.wi_minmax.numel()
                + 2 * self.wo_minmax.numel())

    workspace = _workspace

    def forward(self, x, token_expert, y=None):
        """y[t] = wo_e(relu(wi_e(x[t]))), e = token_expert[t]; tokens with a
        negative expert keep their input.  x bf16 [T, d_model], token_expert
        int32 [T]."""
        dev = self.device
        _lib.check_faults()       # what earlier launches reported (host memory, no sync)
        p_x = _need(x, torch.bfloat16, 'x', dev, dim=2)
        tokens = x.shape[0]
        if x.shape[1] != self.d_model:
            raise ValueError('x must be [T, %d]' % self.d_model)
        p_te = _need(token_expert, torch.int32, 'token_expert', dev, numel=tokens)
        if y is None:
            y = torch.empty_like(x)
        if tokens == 0:
            return y
        p_y = _need(y, torch.bfloat16, 'y', dev, numel=x.numel())
        ws = self.workspace(tokens)
        with _on_device(dev):
            _lib.check(_lib.load().sub1_moe_grouped(
                ctypes.byref(self._c), p_te, p_x, p_y, tokens, ws.data_ptr(),
                ws.numel(), _stream()))
        return y

    def can_prepare(self):
        """Whether the fast layout takes these shapes (it also wants the fixed
        dictionary, which prepare() itself checks)."""
        return max(self.d_model, self.d_ff) <= PREPARED_MAX_WIDTH

    def prepare(self):
        """The fast form of this stack (see PreparedStack); the stack itself
        is left as it is and is not referenced by the result."""
        return PreparedStack(self)

    def launch_faults(self, tokens):
        """(waits that gave up, tokens whose expert id was >= experts and were
        passed through) in the forwards on this stream since the last call of
        this method; both 0 when all is well.  Reads the control words of the
        workspace, synchronising.  A wait that gave up is also reported,
        sticky, by check_faults() and by the next forward()."""
        return _fault_delta(self, tokens)

    check_faults = staticmethod(_lib.check_faults)


class PreparedStack:
    """An ExpertStack decoded once into the form the GPU streams at full width:
    every row's non-zero weights as 7-bit gap entries, rows ordered by length,
    64-row slices, entries interleaved 8 bytes per lane; the kernels keep only
    the activations in LDS.  `forward` has the semantics of
    ExpertStack.forward; a row's fp32 sum is taken in the stream's own order,
    so outputs agree with it to rounding, not to the bit."""

    def __init__(self, stack):
        lib = _lib.load()
        self._make(stack.device, stack.experts, stack.d_model, stack.d_ff,
                   lambda *a: lib.sub1_moe_prepare_layout(ctypes.byref(stack._c), *a),
                   lambda *a: lib.sub1_moe_prepare_codes(ctypes.byref(stack._c), *a))

    @classmethod
    def from_layers(cls, dec, wi_layers, wo_layers):
        """Prepared straight from per-expert (w_comp, row_off, ter_minmax)
        triples, as the experts' Sub1Linear modules hold them: nothing is
        stacked first, the triples are only read."""
        lib = _lib.load()
        dev = dec.device
        experts = len(wi_layers)
        if experts < 1 or len(wo_layers) != experts:
            raise ValueError('as many wi as wo layers, at least one')
        d_ff = wi_layers[0][1].numel() - 1
        d_model = wo_layers[0][1].numel() - 1
        tables = []
        for layers, rows in ((wi_layers, d_ff), (wo_layers, d_model)):
            columns = ([], [], [])
            for w_comp, row_off, minmax in layers:
                columns[0].append(_need(w_comp, torch.int16, 'w_comp', dev))
                columns[1].append(_need(row_off, torch.int32, 'row_off', dev, numel=rows + 1))
                columns[2].append(_need(minmax, torch.bfloat16, 'ter_minmax', dev, numel=2 * rows))
            tables.append([torch.tensor(c, dtype=torch.int64).to(dev) for c in columns])
        (wi_c, wi_r, wi_m), (wo_c, wo_r, wo_m) = tables
        c_layers = _lib.MoeLayers(
            _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS), wi_c.data_ptr(), wo_c.data_ptr(),
            wi_r.data_ptr(), wo_r.data_ptr(), wi_m.data_ptr(), wo_m.data_ptr(), experts, d_model, d_ff)
        self = cls.__new__(cls)
        self._make(dev, experts, d_model, d_ff,
                   lambda *a: lib.sub1_moe_prepare_layout_from_layers(ctypes.byref(c_layers), *a),
                   lambda *a: lib.sub1_moe_prepare_codes_from_layers(ctypes.byref(c_layers), *a))
        return self

    def entry_counts(self):
        """(entries a sweep of all experts walks, entries of the rows
        themselves): the difference is what the stream spends on padding rows
        to the length of their slice."""
        walked, in_rows = ctypes.c_int64(), ctypes.c_int64()
        with _on_device(self.device):
            _lib.check(_lib.load().sub1_moe_prepared_entry_counts(
                ctypes.byref(self._c), ctypes.byref(walked), ctypes.byref(in_rows), _stream()))
        return walked.value, in_rows.value

    def _make(self, dev, experts, d_model, d_ff, layout, codes):
        lib = _lib.load()
        self.device = dev
        self.experts, self.d_model, self.d_ff = experts, d_model, d_ff
        meta_bytes = lib.sub1_moe_prepared_meta_bytes(experts, d_model, d_ff)
        if meta_bytes <= 0:
            raise ValueError('bad stack dimensions')
        self.meta = torch.empty(meta_bytes, dtype=torch.uint8, device=dev)
        self._c = _lib.MoePrepared()
        with _on_device(dev):
            _lib.check(layout(self.meta.data_ptr(), meta_bytes, ctypes.byref(self._c), _stream()))
            self.code_bytes = self._c.code_bytes
            self.stream_bytes = self._c.total_chunks * 512     # without the checkpoints
            self.codes = torch.empty(max(self.code_bytes, 256), dtype=torch.uint8, device=dev)
            self._c.codes = self.codes.data_ptr()
            _lib.check(codes(ctypes.byref(self._c), _stream()))
        self._ws = {}
        self._ws_epoch = {}  # per workspace: fault_epoch() when it was last zeroed
        self._seen = {}      # per workspace: the fault counts launch_faults() last returned from

    workspace = _workspace

    def forward(self, x, token_expert, y=None):
        dev = self.device
        _lib.check_faults()       # what earlier launches reported (host memory, no sync)
        p_x = _need(x, torch.bfloat16, 'x', dev, dim=2)
        tokens = x.shape[0]
        if x.shape[1] != self.d_model:
            raise ValueError('x must be [T, %d]' % self.d_model)
        p_te = _need(token_expert, torch.int32, 'token_expert', dev, numel=tokens)
        if y is None:
            y = torch.empty_like(x)
        if tokens == 0:
            return y
        p_y = _need(y, torch.bfloat16, 'y', dev, numel=x.numel())
        ws = self.workspace(tokens)
        with _on_device(dev):
            _lib.check(_lib.load().sub1_moe_grouped_prepared(
                ctypes.byref(self._c), p_te, p_x, p_y, tokens, ws.data_ptr(), ws.numel(),
                _stream()))
        return y

    def launch_faults(self, tokens):
        """As ExpertStack.launch_faults."""
        return _fault_delta(self, tokens)

    check_faults = staticmethod(_lib.check_faults)

    def decode(self, expert, projection):
        """uint8 [rows, width]: the symbols of one matrix (projection 0 = wi,
        1 = wo) read back from the prepared stream."""
        rows, width = (self.d_ff, self.d_model) if projection == 0 else (self.d_model, self.d_ff)
        out = torch.empty(rows, width, dtype=torch.uint8, device=self.device)
        with _on_device(self.device):
            _lib.check(_lib.load().sub1_moe_prepared_decode(
                ctypes.byref(self._c), expert, projection, out.data_ptr(), _stream()))
        return out


class PreparedMatrix:
    """Compressed matrices of one shape copied into the fast layout;
    `matvec_tokens(x, y)` does y[t] += W x[t] like sub1matvec_tokens, in one
    launch over the prepared stream.

    One matrix: the three buffers of a Sub1Linear.  Several: pass lists of
    equally shaped buffers (or stacked tensors plus `code_base`, int64 [count],
    the first codeword of each matrix in `w_comp`); `matvec_tokens` then takes
    `token_matrix`, int32 [T], the matrix each token uses."""

    def __init__(self, dec, w_comp, row_off, ter_minmax, width, code_base=None):
        lib = _lib.load()
        dev = dec.device
        if isinstance(w_comp, (list, tuple)):
            sizes = torch.tensor([0] + [t.numel() for t in w_comp], dtype=torch.int64)
            code_base = sizes.cumsum(0)[:-1].to(dev)
            w_comp, row_off, ter_minmax = (torch.cat(list(v)) for v in (w_comp, row_off, ter_minmax))
        count = 1 if code_base is None else code_base.numel()
        if row_off.numel() % count:
            raise ValueError('row_off does not hold %d equal parts' % count)
        height = row_off.numel() // count - 1
        self.device, self.count, self.height, self.width = dev, count, height, width
        src = _lib.MatrixSet(
            _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS),
            _need(w_comp, torch.int16, 'w_comp', dev),
            None if code_base is None else _need(code_base, torch.int64, 'code_base', dev),
            _need(row_off, torch.int32, 'row_off', dev, numel=count * (height + 1)),
            _need(ter_minmax, torch.bfloat16, 'ter_minmax', dev, numel=count * 2 * height),
            count, height, width)
        meta_bytes = lib.sub1_matrix_prepared_meta_bytes(count, height, width)
        if meta_bytes <= 0:
            raise ValueError('bad matrix dimensions')
        self.meta = torch.empty(meta_bytes, dtype=torch.uint8, device=dev)
        self._c = _lib.MatrixPrepared()
        with _on_device(dev):
            _lib.check(lib.sub1_matrix_prepare_layout(ctypes.byref(src), self.meta.data_ptr(),
                                                      meta_bytes, ctypes.byref(self._c), _stream()))
            self.codes = torch.empty(max(self._c.code_bytes, 256), dtype=torch.uint8, device=dev)
            self._c.codes = self.codes.data_ptr()
            _lib.check(lib.sub1_matrix_prepare_codes(ctypes.byref(src), ctypes.byref(self._c),
                                                     _stream()))

    def matvec_tokens(self, x, y, token_matrix=None):
        dev = self.device
        p_x = _need(x, torch.bfloat16, 'x', dev, dim=2)
        p_y = _need(y, torch.bfloat16, 'y', dev, dim=2)
        tokens = x.shape[0]
        if x.shape[1] != self.width or y.shape != (tokens, self.height):
            raise ValueError('x must be [T, %d] and y [T, %d]' % (self.width, self.height))
        if token_matrix is None and self.count > 1:
            raise ValueError('token_matrix is required with %d matrices' % self.count)
        p_tm = None if token_matrix is None else _need(token_matrix, torch.int32, 'token_matrix',
                                                       dev, numel=tokens)
        if tokens == 0:
            return
        with _on_device(dev):
            _lib.check(_lib.load().sub1_matvec_prepared(
                ctypes.byref(self._c), p_tm, p_x, self.width, p_y, self.height, tokens, _stream()))

    def decode(self, matrix=0):
        """uint8 [height, width]: the symbols of one matrix read back from the
        prepared stream."""
        out = torch.empty(self.height, self.width, dtype=torch.uint8, device=self.device)
        with _on_device(self.device):
            _lib.check(_lib.load().sub1_matrix_prepared_decode(
                ctypes.byref(self._c), matrix, out.data_ptr(), _stream()))
        return out


class TiledMatrix:
    """Compressed matrices of one shape copied into the tile form that the
    matrix cores multiply from; `matvec_tokens(x, y)` does y[t] += W x[t] for
    all tokens of x [T, width] in one launch, the weights decoded once per
    tile of 64 tokens (made for sequences: from a few dozen tokens on it beats
    walking the non-zeros per token; results agree with the other paths to
    rounding, not to the bit).  Arguments as PreparedMatrix."""

    def __init__(self, dec, w_comp, row_off, ter_minmax, width, code_base=None):
        lib = _lib.load()
        dev = dec.device
        if isinstance(w_comp, (list, tuple)):
            sizes = torch.tensor([0] + [t.numel() for t in w_comp], dtype=torch.int64)
            code_base = sizes.cumsum(0)[:-1].to(dev)
            w_comp, row_off, ter_minmax = (torch.cat(list(v)) for v in (w_comp, row_off, ter_minmax))
        count = 1 if code_base is None else code_base.numel()
        if row_off.numel() % count:
            raise ValueError('row_off does not hold %d equal parts' % count)
        height = row_off.numel() // count - 1
        self.device, self.count, self.height, self.width = dev, count, height, width
        src = _lib.MatrixSet(
            _need(dec, torch.int32, 'dec', numel=_lib.DEC_WORDS),
            _need(w_comp, torch.int16, 'w_comp', dev),
            None if code_base is None else _need(code_base, torch.int64, 'code_base', dev),
            _need(row_off, torch.int32, 'row_off', dev, numel=count * (height + 1)),
            _need(ter_minmax, torch.bfloat16, 'ter_minmax', dev, numel=count * 2 * height),
            count, height, width)
        meta_bytes = lib.sub1_tiles_meta_bytes(count, height, width)
        if meta_bytes <= 0:
            raise ValueError('bad matrix dimensions')
        self.meta = torch.empty(meta_bytes, dtype=torch.uint8, device=dev)
        self._c = _lib.Tiles()
        with _on_device(dev):
            _lib.check(lib.sub1_tiles_layout(ctypes.byref(src), self.meta.data_ptr(), meta_bytes,
                                             ctypes.byref(self._c), _stream()))
            self.entries = torch.empty(max(self._c.entry_bytes, 256), dtype=torch.uint8, device=dev)
            self._c.entries = self.entries.data_ptr()
            _lib.check(lib.sub1_tiles_entries(ctypes.byref(src), ctypes.byref(self._c), _stream()))

    def matvec_tokens(self, x, y, matrix=0):
        dev = self.device
        p_x = _need(x, torch.bfloat16, 'x', dev, dim=2)
        p_y = _need(y, torch.bfloat16, 'y', dev, dim=2)
        tokens = x.shape[0]
        if x.shape[1] != self.width or y.shape != (tokens, self.height):
            raise ValueError('x must be [T, %d] and y [T, %d]' % (self.width, self.height))
        if tokens == 0:
            return
        with _on_device(dev):
            _lib.check(_lib.load().sub1_matvec_tiles(
                ctypes.byref(self._c), matrix, p_x, self.width, p_y, self.height, tokens, _stream()))

    def decode(self, matrix=0):
        """uint8 [height, width]: the symbols of one matrix read back from the
        tile form."""
        out = torch.empty(self.height, self.width, dtype=torch.uint8, device=self.device)
        with _on_device(self.device):
            _lib.check(_lib.load().sub1_tiles_decode(ctypes.byref(self._c), matrix, out.data_ptr(),
                                                     _stream()))
        return out
