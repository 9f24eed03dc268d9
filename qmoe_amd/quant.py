"""Ternary quantiser front end of the reference (quant.py:24-28, 31-75): the
round-to-nearest rule that turns a dense matrix into rows of {row min, 0,
row max}, which is what `Sub1Linear.make` packs.  Only the ternary setting
(`bits == 1.5`) of the reference's `Quantizer` feeds the compressed layer, so
only that one exists here; the integer grids belong to the GPTQ pipeline.

Plain tensor arithmetic (torch, any device): this runs once per matrix,
offline, and is not part of the decode path.
"""
import torch
import torch.nn as nn


def quantize(x, scale, zero, maxq):
    """Reference quant.py:24-28, ternary branch (`maxq < 0`): `scale` carries
    the row maximum and `zero` the row minimum; a value becomes the maximum
    if it exceeds half of it, the minimum if it is below half of it, else 0."""
    if maxq >= 0:
        raise NotImplementedError('only the ternary grid (bits = 1.5) is implemented')
    return (x > scale / 2).float() * scale + (x < zero / 2).float() * zero


class Quantizer(nn.Module):
    """Reference quant.py:30-75 for `bits == 1.5`."""

    def configure(self, bits, sym=False):
        if bits != 1.5:
            raise NotImplementedError('only the ternary grid (bits = 1.5) is implemented')
        self.maxq = torch.tensor(-1)   # the reference's marker for ternary
        self.sym = sym

    def find_params(self, x):
        """Per row of the last dimension: maximum (clamped to >= 0) into
        `scale`, minimum (clamped to <= 0) into `zero`; `sym` makes rows with
        a negative entry symmetric; an all-zero row gets (-1, +1)
        (reference quant.py:41-72)."""
        dev = x.device
        self.maxq = self.maxq.to(dev)
        floor = torch.zeros(x.shape[:-1], device=dev, dtype=x.dtype)
        xmin = torch.minimum(x.min(-1)[0], floor)
        xmax = torch.maximum(x.max(-1)[0], floor)
        if self.sym:
            xmax = torch.maximum(torch.abs(xmin), xmax)
            neg = xmin < 0
            if torch.any(neg):
                xmin[neg] = -xmax[neg]
        dead = (xmin == 0) & (xmax == 0)
        xmin[dead] = -1
        xmax[dead] = +1
        self.scale = xmax.unsqueeze(-1)
        self.zero = xmin.unsqueeze(-1)

    def ready(self):
        return hasattr(self, 'scale')

    def quantize(self, x):
        if self.ready():
            return quantize(x, self.scale, self.zero, self.maxq)
        return x


def ternarize(w, sym=False):
    """Round-to-nearest ternary version of a dense [H, W] matrix, ready for
    `Sub1Linear.make`."""
    q = Quantizer()
    q.configure(1.5, sym=sym)
    q.find_params(w.float())
    return q.quantize(w.float())
