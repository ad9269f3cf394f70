"""JoinTable / AddTable / ConcatTable (reference: sparseconvnet/tables.py:13-48) and the
pass-through branch of a ConcatTable, Identity (sparseconvnet/identity.py)."""
import torch

from . import SCN, incremental
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf


class JoinTable(torch.nn.Sequential):
    """Concatenates feature planes.  Each input is written straight into its column slice of
    one output matrix (no torch.cat)."""

    def __init__(self, *args):
        torch.nn.Sequential.__init__(self, *args)
        self._state = StateBuf()

    def forward(self, input, increment=False):
        output = SparseConvNetTensor(None, input[0].metadata, input[0].spatial_size)
        n = input[0].features.size(0)
        C = sum(i.features.size(1) for i in input)
        kind = incremental.kind(increment)
        if kind == "residual":  # a frame's rows only; the cached output is left alone
            increment = False
            out = torch.empty((n, C), dtype=torch.float32, device=input[0].features.device)
        elif increment:
            d = input[0].dirty
            for i in input[1:]:
                d = incremental.union(d, i.dirty)
            rows, count = d.rows(d.scale.order.t)
            output.dirty = d
            out = self._state.grow(n, keep=min(n, self._state.buf.size(0)))
        else:
            out = self._state.new(n, C, input[0].features)
        c0 = 0
        for i in input:
            c = i.features.size(1)
            if n:
                if increment:
                    SCN.copy_rows(i.features, out[:, c0:c0 + c], rows, count, d.n_upper)
                else:
                    SCN.copy_rows(i.features, out[:, c0:c0 + c], None, None, n)
            c0 += c
        output.features = out
        return output

    def input_spatial_size(self, out_size):
        return out_size


class AddTable(torch.nn.Sequential):
    def __init__(self, *args):
        torch.nn.Sequential.__init__(self, *args)
        self._state = StateBuf()

    def forward(self, input, increment=False):
        output = SparseConvNetTensor(None, input[0].metadata, input[0].spatial_size)
        n, C = input[0].features.shape
        rows = count = None
        n_rows = n
        kind = incremental.kind(increment)
        if kind == "residual":
            increment = False
            out = torch.empty((n, C), dtype=torch.float32, device=input[0].features.device)
        elif increment:
            d = input[0].dirty
            for i in input[1:]:
                d = incremental.union(d, i.dirty)
            rows, count = d.rows(d.scale.order.t)
            n_rows = d.n_upper
            output.dirty = d
            out = self._state.grow(n, keep=min(n, self._state.buf.size(0)))
        else:
            out = self._state.new(n, C, input[0].features)
        if n and len(input) == 1:  # a sum of one term (the reference sums any number of inputs >= 1)
            SCN.copy_rows(input[0].features, out, rows, count, n_rows)
        elif n:
            SCN.add_rows(input[0].features, input[1].features, out, rows, count, n_rows)
            for i in input[2:]:
                SCN.add_rows(out, i.features, out, rows, count, n_rows)
        output.features = out
        return output

    def input_spatial_size(self, out_size):
        return out_size


class ConcatTable(torch.nn.Sequential):
    def __init__(self, *args):
        torch.nn.Sequential.__init__(self, *args)

    def forward(self, input, increment=False):
        return [module(input, increment) for module in self._modules.values()]

    def add(self, module):
        self._modules[str(len(self._modules))] = module
        return self

    def input_spatial_size(self, out_size):
        return self._modules['0'].input_spatial_size(out_size)


class Identity(torch.nn.Module):
    """The skip branch of a residual block or of a U-Net scale: hands its input on, whatever the
    kind of forward."""

    def forward(self, input, increment=False):
        return input

    def input_spatial_size(self, out_size):
        return out_size
