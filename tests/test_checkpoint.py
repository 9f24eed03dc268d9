"""The checkpoint directory format (reference sub1.py:169-214 writer,
sub1.py:250-292 reader): file names, key names, sizes, round trip.  Layers are
packed on the CPU with the oracle's encoder, so no GPU is needed."""
import os

import numpy as np
import pytest
import torch

from oracle import sub1_oracle as so
from qmoe_amd import checkpoint, sub1


def packed_layer(oracle, height, width, seed):
    t, mm = so.synthetic_ternary(height, width, 0.85, seed)
    codes, row_off = oracle.encode(t)
    layer = sub1.Sub1Linear(height, codes.size)
    layer.w_comp.data = torch.from_numpy(codes.view(np.int16).copy())
    layer.row_off.data = torch.from_numpy(row_off.copy())
    layer.ter_minmax.data = torch.from_numpy(mm.view(np.int16).copy()).view(torch.bfloat16)
    return layer


def expert_name(root, block, j):
    return '%s.block.%d.layer.%d.mlp.experts.expert_%d' % (root, block, 1 if root == 'encoder' else 2, j)


@pytest.fixture()
def written(tmp_path, oracle):
    d_model, d_ff = 32, 64
    experts = {}
    mgr = checkpoint.Sub1CheckpointManager(
        str(tmp_path), config={'d_model': d_model, 'd_ff': d_ff, 'num_experts': 3},
        noexp={'shared.weight': torch.ones(4, d_model), 'step': torch.tensor(3)})
    seed = 0
    for root, block in (('encoder', 1), ('decoder', 3)):
        for j in (2, 0, 1):                       # out of order on purpose
            wi = packed_layer(oracle, d_ff, d_model, seed)
            wo = packed_layer(oracle, d_model, d_ff, seed + 1)
            seed += 2
            name = expert_name(root, block, j)
            experts[name] = (wi, wo)
            mgr.add_expert(name, wi, wo)
        mgr.save_experts()
    mgr.finalize()
    return str(tmp_path), experts


def test_directory_layout_and_keys(written):
    path, experts = written
    assert sorted(os.listdir(path)) == ['config.json', 'exp00.pt', 'exp01.pt', 'noexp.pt', 'sizes.pt']
    sizes = torch.load(os.path.join(path, 'sizes.pt'), weights_only=True)
    name = expert_name('encoder', 1, 0)
    assert sizes[name + '.wi'] == experts[name][0].w_comp.numel()
    assert sizes[name + '.wo'] == experts[name][1].w_comp.numel()
    exp0 = torch.load(os.path.join(path, 'exp00.pt'), weights_only=True)
    assert set(k[len(name) + 1:] for k in exp0 if k.startswith(name + '.')) == {
        'wi.w_comp', 'wi.row_off', 'wi.ter_minmax', 'wi.weight',
        'wo.w_comp', 'wo.row_off', 'wo.ter_minmax', 'wo.weight'}
    assert exp0[name + '.wi.w_comp'].dtype == torch.int16
    assert exp0[name + '.wi.row_off'].dtype == torch.int32
    assert exp0[name + '.wi.ter_minmax'].dtype == torch.bfloat16
    assert exp0[name + '.wi.weight'].numel() == 0
    noexp = torch.load(os.path.join(path, 'noexp.pt'), weights_only=True)
    assert noexp['shared.weight'].dtype == torch.bfloat16 and int(noexp['step']) == 3
    import json
    assert json.load(open(os.path.join(path, 'config.json')))['torch_dtype'] == 'bfloat16'


def test_round_trip_in_expert_order(written):
    path, experts = written
    layers = checkpoint.load_expert_layers(path)
    assert sorted(layers) == ['decoder.block.3.layer.2.mlp', 'encoder.block.1.layer.1.mlp']
    for layer_name, pairs in layers.items():
        assert len(pairs) == 3
        for j, (wi, wo) in enumerate(pairs):
            src_wi, src_wo = experts['%s.experts.expert_%d' % (layer_name, j)]
            for got, src in ((wi, src_wi), (wo, src_wo)):
                assert torch.equal(got.w_comp, src.w_comp)
                assert torch.equal(got.row_off, src.row_off)
                assert torch.equal(got.ter_minmax.view(torch.int16), src.ter_minmax.view(torch.int16))


def test_reader_rejects_damage(written):
    path, _ = written
    sizes = torch.load(os.path.join(path, 'sizes.pt'), weights_only=True)
    key = expert_name('encoder', 1, 1) + '.wo'
    bad = dict(sizes)
    bad[key] += 1
    torch.save(bad, os.path.join(path, 'sizes.pt'))
    with pytest.raises(ValueError):
        checkpoint.load_expert_layers(path)
    bad = {k: v for k, v in sizes.items() if not k.startswith(expert_name('decoder', 3, 1))}
    torch.save(bad, os.path.join(path, 'sizes.pt'))
    with pytest.raises(ValueError):
        checkpoint.load_expert_layers(path)          # expert 1 of 0..2 missing


def test_prepared_only_reader_checks_the_directory_first(written):
    """The streaming reader reads sizes.pt before any expert file: entries
    that are not experts' wi / wo, and expert indices with holes, raise before
    anything is put on a GPU (none is needed to get that far)."""
    path, _ = written
    sizes = torch.load(os.path.join(path, 'sizes.pt'), weights_only=True)
    bad = {k: v for k, v in sizes.items() if not k.startswith(expert_name('decoder', 3, 1))}
    torch.save(bad, os.path.join(path, 'sizes.pt'))
    with pytest.raises(ValueError, match='indices'):
        checkpoint.load_prepared_experts(path, 'cpu')
    bad = dict(sizes)
    bad['encoder.block.1.layer.1.mlp.router.classifier'] = 3
    torch.save(bad, os.path.join(path, 'sizes.pt'))
    with pytest.raises(ValueError, match='unexpected'):
        checkpoint.load_prepared_experts(path, 'cpu')


def test_writer_rejects_other_names(tmp_path, oracle):
    mgr = checkpoint.Sub1CheckpointManager(str(tmp_path))
    layer = packed_layer(oracle, 8, 8, 1)
    with pytest.raises(ValueError):
        mgr.add_expert('encoder.block.0.layer.1.mlp.wi', layer, layer)
