"""FasterMLP's reading of a Switch top-1 router's outputs (reference
sub1.py:310 unpacks transformers 4.28's `(mask, probs, logits)`), on the CPU:
the router class of the installed transformers built from a config (nothing is
fetched), and the 4.28 tuple restated by hand."""
import pytest
import torch


def hand_router(hidden, weight, capacity):
    """What SwitchTransformersTop1Router computes (fp32 softmax of a linear
    classifier, one-hot argmax, capacity by position in the sequence)."""
    logits = hidden.float() @ weight.float().t()
    probs = torch.softmax(logits, dim=-1)
    index = probs.argmax(dim=-1)
    mask = torch.nn.functional.one_hot(index, weight.shape[0])
    mask = mask * (torch.cumsum(mask, dim=-2) <= capacity)
    return mask, probs.max(dim=-1).values.unsqueeze(-1), logits


def test_transformers_428_order():
    from qmoe_amd.sub1 import _router_outputs
    g = torch.Generator().manual_seed(3)
    hidden = torch.randn((2, 9, 16), generator=g)
    weight = torch.randn((5, 16), generator=g)
    mask, probs, logits = hand_router(hidden, weight, capacity=2)
    got = _router_outputs((mask, probs, logits), 5)
    assert got[0] is mask and got[1] is probs and got[2] is logits
    assert int((mask.sum(-1) == 0).sum()) > 0          # the capacity limit dropped tokens


def test_single_expert_and_bad_tuples():
    from qmoe_amd.sub1 import _router_outputs
    mask = torch.ones((3, 4, 1), dtype=torch.int64)
    probs = torch.ones((3, 4, 1))
    logits = torch.zeros((3, 4, 1))
    got = _router_outputs((mask, probs, logits), 1)
    assert got[0] is mask and got[1] is probs and got[2] is logits
    with pytest.raises(ValueError):
        _router_outputs((probs, logits, logits), 1)                    # no mask
    with pytest.raises(ValueError):
        _router_outputs((mask, probs), 1)
    with pytest.raises(ValueError):
        _router_outputs((torch.ones((3, 4, 7), dtype=torch.int64), probs, logits), 5)


@pytest.mark.parametrize('leading', [(2, 7), (14,)])
def test_installed_transformers_router(leading):
    """The installed transformers' own router, from a config: whatever tuple it
    returns, the mask, probabilities and route FasterMLP derives are those of
    the router restated by hand."""
    pytest.importorskip('transformers')
    from transformers.models.switch_transformers import modeling_switch_transformers as hf
    from qmoe_amd.sub1 import _router_outputs
    cfg = hf.SwitchTransformersConfig(d_model=32, d_ff=64, num_experts=6, expert_capacity=64,
                                      num_layers=2, num_sparse_encoder_layers=1, num_heads=2,
                                      d_kv=16, vocab_size=64, router_jitter_noise=0.0)
    torch.manual_seed(5)
    router = hf.SwitchTransformersTop1Router(cfg).eval()
    hidden = torch.randn(leading + (32,))
    with torch.no_grad():
        mask, probs, _ = _router_outputs(router(hidden), cfg.num_experts)
    want_mask, want_probs, _ = hand_router(hidden, router.classifier.weight.detach(), 64)
    assert mask.shape == leading + (6,) and probs.shape == leading + (1,)
    assert torch.equal(mask.to(torch.int64), want_mask)
    assert torch.allclose(probs.float(), want_probs, rtol=1e-6, atol=0)
    route = torch.where(mask.any(dim=-1), mask.argmax(dim=-1), -1)
    assert torch.equal(route, want_mask.argmax(dim=-1))


def test_output_form_follows_the_wrapped_module():
    """transformers 5.x's sparse MLP returns a tensor, 4.28's a pair; FasterMLP
    returns what the block around the wrapped module expects."""
    import types
    import torch.nn as nn
    from qmoe_amd import sub1

    class TensorMLP(nn.Module):
        def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
            return hidden_states

    class PairMLP(nn.Module):
        def forward(self, hidden_states):
            return hidden_states, (None, None)

    for cls, pair in ((TensorMLP, False), (PairMLP, True)):
        mlp = cls()
        mlp.router = nn.Identity()
        mlp.experts = nn.ModuleDict()
        assert sub1.FasterMLP(mlp).router_outputs is pair
    loose = types.SimpleNamespace(router=nn.Identity(), experts=nn.ModuleDict())
    assert sub1.FasterMLP(loose).router_outputs is True
    assert sub1.FasterMLP(loose, router_outputs=False).router_outputs is False
