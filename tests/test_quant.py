"""The ternary quantiser front end (reference quant.py:24-28, 41-72) against
answers worked out by hand from the reference's rule: max and min per row
(clamped at zero), value -> max if above max/2, min if below min/2, else 0."""
import numpy as np
import pytest
import torch

from qmoe_amd import quant


def test_known_answers():
    w = torch.tensor([[0.9, 0.5, 0.44, 0.0, -0.1, -0.21, -0.4],     # max .9, min -.4
                      [0.2, 0.1, 0.05, 0.3, 0.16, 0.15, 0.0],       # no negative: min 0
                      [-1.0, -0.5, -0.51, 0.0, -2.0, -0.99, -1.01],  # no positive: max 0
                      [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]])         # dead row: (-1, +1)
    q = quant.Quantizer()
    q.configure(1.5)
    assert not q.ready() and q.quantize(w) is w
    q.find_params(w)
    assert q.ready() and int(q.maxq) == -1
    assert q.scale.flatten().tolist() == pytest.approx([0.9, 0.3, 0.0, 1.0])
    assert q.zero.flatten().tolist() == pytest.approx([-0.4, 0.0, -2.0, -1.0])
    got = q.quantize(w)
    want = torch.tensor([[0.9, 0.9, 0.0, 0.0, 0.0, -0.4, -0.4],     # .5 > .45; .44 < .45; -.21 < -.2
                         [0.3, 0.0, 0.0, 0.3, 0.3, 0.0, 0.0],       # threshold .15 is exclusive
                         [0.0, 0.0, 0.0, 0.0, -2.0, 0.0, -2.0],     # threshold -1 is exclusive
                         [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0]])
    assert torch.allclose(got, want)


def test_symmetric_rows():
    w = torch.tensor([[0.2, -1.0, 0.6, 0.4],      # has a negative: range becomes (-1, 1)
                      [0.2, 0.8, 0.5, 0.3]])      # none: min stays 0
    q = quant.Quantizer()
    q.configure(1.5, sym=True)
    q.find_params(w)
    assert q.scale.flatten().tolist() == pytest.approx([1.0, 0.8])
    assert q.zero.flatten().tolist() == pytest.approx([-1.0, 0.0])
    assert torch.allclose(q.quantize(w), torch.tensor([[0.0, -1.0, 1.0, 0.0],
                                                       [0.0, 0.8, 0.8, 0.0]]))


def test_rows_take_three_values_and_batched_shapes():
    g = torch.Generator().manual_seed(3)
    w = torch.randn((4, 32, 50), generator=g)
    out = quant.ternarize(w)
    assert out.shape == w.shape
    hi = w.max(-1, keepdim=True)[0]
    lo = w.min(-1, keepdim=True)[0]
    assert torch.all((out == 0) | (out == hi) | (out == lo))
    # idempotent: a ternary matrix is its own quantisation
    assert torch.equal(quant.ternarize(out), out)
    # numpy restatement of the decision rule on the same numbers
    wn, hn, ln = w.numpy(), hi.numpy(), lo.numpy()
    ref = np.where(wn > hn / 2, hn, 0) + np.where(wn < ln / 2, ln, 0)
    assert np.array_equal(out.numpy(), ref.astype(np.float32))


def test_other_grids_are_refused():
    q = quant.Quantizer()
    with pytest.raises(NotImplementedError):
        q.configure(2)
    with pytest.raises(NotImplementedError):
        quant.quantize(torch.zeros(2, 2), torch.ones(2, 1), torch.ones(2, 1), torch.tensor(3))
