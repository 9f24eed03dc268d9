"""The on-disk form of a compressed model's experts, as the reference writes
and reads it (sub1.py:169-214 `Sub1CheckpointManager`, sub1.py:217-292
`load_sub1`):

    config.json   model configuration (written by the caller's config object)
    noexp.pt      state dict of everything that is not an expert
    expNN.pt      state dicts of packed experts, keys
                  '<expert name>.wi.w_comp' / '.row_off' / '.ter_minmax' /
                  '.weight' and the same under '.wo.'
    sizes.pt      {'<expert name>.wi': codewords, '<expert name>.wo': ...}

with expert names '<encoder|decoder>.block.<i>.layer.<1|2>.mlp.experts.expert_<j>'
(reference switch.py:424-426).  The writer here takes packed layers directly
(no HuggingFace model needed); the reader returns, per MoE layer, the experts'
layers in index order, ready for `Sub1Experts` / `FasterMLP`, or, for models
too large to hold twice, the layers already prepared with the packed form
dropped (`load_prepared_experts`).

Files are read with `torch.load(..., weights_only=True)`: tensors and plain
containers only.
"""
import json
import os
import re

import torch

from . import sub1

_EXPERT = re.compile(r'^(?P<layer>.+\.mlp)\.experts\.expert_(?P<index>\d+)$')
_FILES_SKIPPED = ('sizes.pt', 'config.json', 'README.md', '.gitattributes', '.git')


class Sub1CheckpointManager:
    """Writer (reference sub1.py:169-214).  `config` is a plain dict (or
    anything with `to_dict()`), `noexp` the state dict of the non-expert
    parameters; either may be None when only experts are stored."""

    def __init__(self, path, config=None, noexp=None):
        os.makedirs(path, exist_ok=True)
        self.path = path
        if config is not None:
            cfg = dict(config.to_dict() if hasattr(config, 'to_dict') else config)
            cfg['torch_dtype'] = 'bfloat16'          # reference sub1.py:186
            with open(os.path.join(path, 'config.json'), 'w') as f:
                json.dump(cfg, f, indent=2, sort_keys=True)
        if noexp is not None:
            torch.save({k: (v.bfloat16() if v.is_floating_point() else v).cpu()
                        for k, v in noexp.items()}, os.path.join(path, 'noexp.pt'))
        self.sd_exp = [{}]
        self.sizes = {}

    def add_expert(self, name, wi, wo):
        """Buffer one expert's packed layers (reference sub1.py:194-204, which
        packs `expert.wi/wo` with Sub1Linear.make first; here they arrive
        packed)."""
        if not _EXPERT.match(name):
            raise ValueError('not an expert name: %r' % name)
        for tag, layer in (('wi', wi), ('wo', wo)):
            for n, p in layer.state_dict().items():
                self.sd_exp[-1]['%s.%s.%s' % (name, tag, n)] = p.cpu()
            self.sizes['%s.%s' % (name, tag)] = layer.w_comp.numel()

    def save_experts(self):
        """Write the buffered experts to the next expNN.pt (sub1.py:207-210)."""
        torch.save(self.sd_exp[-1], os.path.join(self.path, 'exp%02d.pt' % (len(self.sd_exp) - 1)))
        self.sd_exp[-1] = None
        self.sd_exp.append({})

    def finalize(self):
        """Write sizes.pt (sub1.py:213-214)."""
        if self.sd_exp[-1]:
            self.save_experts()
        torch.save(self.sizes, os.path.join(self.path, 'sizes.pt'))


def load_expert_layers(path, device=None):
    """{layer name: [(wi, wo) Sub1Linear pairs in expert order]} from a
    checkpoint directory.  Layers are allocated from sizes.pt and filled from
    the expNN.pt files, as load_sub1 does (sub1.py:250, 262, 284-292).
    Raises if an expert is incomplete or an index is missing."""
    sizes = torch.load(os.path.join(path, 'sizes.pt'), weights_only=True)
    tensors = {}
    for filename in sorted(os.listdir(path)):
        if filename in _FILES_SKIPPED or filename == 'noexp.pt' or not filename.endswith('.pt'):
            continue
        tensors.update(torch.load(os.path.join(path, filename), weights_only=True))
    layers = {}
    for key, comp_size in sizes.items():
        name, tag = key.rsplit('.', 1)
        m = _EXPERT.match(name)
        if not m or tag not in ('wi', 'wo'):
            raise ValueError('unexpected entry in sizes.pt: %r' % key)
        try:
            w_comp = tensors[key + '.w_comp']
            row_off = tensors[key + '.row_off']
            ter_minmax = tensors[key + '.ter_minmax']
        except KeyError as err:
            raise ValueError('checkpoint lacks %s' % err.args[0])
        if w_comp.numel() != comp_size or int(row_off[-1]) != comp_size:
            raise ValueError('%s: %d codewords stored, sizes.pt says %d, row_off ends at %d'
                             % (key, w_comp.numel(), comp_size, int(row_off[-1])))
        layer = sub1.Sub1Linear(row_off.numel() - 1, comp_size)
        layer.w_comp.data = w_comp.to(torch.int16)
        layer.row_off.data = row_off.to(torch.int32)
        layer.ter_minmax.data = ter_minmax.to(torch.bfloat16)
        if device is not None:
            layer = layer.to(device)
        layers.setdefault(m.group('layer'), {}).setdefault(int(m.group('index')), {})[tag] = layer
    out = {}
    for layer_name, experts in layers.items():
        pairs = []
        for j in range(len(experts)):
            if j not in experts or set(experts[j]) != {'wi', 'wo'}:
                raise ValueError('%s: expert %d is missing or incomplete' % (layer_name, j))
            pairs.append((experts[j]['wi'], experts[j]['wo']))
        out[layer_name] = pairs
    return out


def load_prepared_experts(path, device):
    """{layer name: Sub1Experts} on `device`, each holding only the prepared
    stream of its experts' weights.  For checkpoints whose packed form and
    prepared form do not fit the GPU side by side: the files are read one at a
    time, a layer is stacked, prepared and its packed tensors dropped as soon
    as its last expert has arrived, so the GPU holds the prepared layers plus
    the experts of layers still incomplete.  Expert counts come from sizes.pt
    (reference sub1.py:250); a layer with experts missing raises at the end."""
    sizes = torch.load(os.path.join(path, 'sizes.pt'), weights_only=True)
    want = {}
    for key in sizes:
        name, tag = key.rsplit('.', 1)
        m = _EXPERT.match(name)
        if not m or tag not in ('wi', 'wo'):
            raise ValueError('unexpected entry in sizes.pt: %r' % key)
        want.setdefault(m.group('layer'), set()).add(int(m.group('index')))
    for layer_name, have in want.items():
        if have != set(range(len(have))):
            raise ValueError('%s: expert indices in sizes.pt are not 0..%d'
                             % (layer_name, len(have) - 1))
    pending, out = {}, {}
    for filename in sorted(os.listdir(path)):
        if filename in _FILES_SKIPPED or filename == 'noexp.pt' or not filename.endswith('.pt'):
            continue
        tensors = torch.load(os.path.join(path, filename), weights_only=True)
        for key in [k for k in tensors if k.endswith('.w_comp')]:
            stem = key[:-len('.w_comp')]
            name, tag = stem.rsplit('.', 1)
            m = _EXPERT.match(name)
            if not m or tag not in ('wi', 'wo') or stem not in sizes:
                raise ValueError('%s holds %r, which sizes.pt does not list' % (filename, key))
            try:
                w_comp, row_off = tensors[key], tensors[stem + '.row_off']
                ter_minmax = tensors[stem + '.ter_minmax']
            except KeyError as err:
                raise ValueError('checkpoint lacks %s' % err.args[0])
            if w_comp.numel() != sizes[stem] or int(row_off[-1]) != sizes[stem]:
                raise ValueError('%s: %d codewords stored, sizes.pt says %d, row_off ends at %d'
                                 % (stem, w_comp.numel(), sizes[stem], int(row_off[-1])))
            layer = sub1.Sub1Linear(row_off.numel() - 1, w_comp.numel())
            layer.w_comp.data = w_comp.to(torch.int16)
            layer.row_off.data = row_off.to(torch.int32)
            layer.ter_minmax.data = ter_minmax.to(torch.bfloat16)
            pending.setdefault(m.group('layer'), {}).setdefault(int(m.group('index')), {})[tag] = \
                layer.to(device)
        del tensors
        for layer_name in list(pending):
            experts = pending[layer_name]
            if len(experts) == len(want[layer_name]) and \
                    all(set(e) == {'wi', 'wo'} for e in experts.values()):
                stacked = sub1.Sub1Experts([experts[j]['wi'] for j in range(len(experts))],
                                           [experts[j]['wo'] for j in range(len(experts))])
                stacked.release_packed()
                out[layer_name] = stacked
                del pending[layer_name]
    if pending or set(out) != set(want):
        missing = sorted(set(want) - set(out))
        raise ValueError('incomplete layers in %s: %s' % (path, ', '.join(missing)))
    return out


def load_expert_stacks(path, device):
    """{layer name: Sub1Experts} on `device`: every MoE layer of the
    checkpoint as one stacked, one-launch module."""
    return {name: sub1.Sub1Experts([p[0] for p in pairs], [p[1] for p in pairs])
            for name, pairs in load_expert_layers(path, device).items()}
