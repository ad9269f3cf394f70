"""NetworkInNetwork, a 1x1 linear layer (reference: sparseconvnet/networkInNetwork.py:59-88)."""
import torch
from torch.nn import Module, Parameter

import sparseconvnet

from . import SCN, incremental
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf, optionalTensor


class NetworkInNetwork(Module):
    def __init__(self, nIn, nOut, bias):
        Module.__init__(self)
        self.nIn = nIn
        self.nOut = nOut
        std = (2.0 / nIn) ** 0.5
        self.weight = Parameter(torch.Tensor(nIn, nOut).normal_(0, std))
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())
        self._state = StateBuf()

    def forward(self, input, increment=False):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn, (self.nIn, input.features.shape)
        output = SparseConvNetTensor(None, input.metadata, input.spatial_size)
        kind = incremental.kind(increment)
        if kind == "residual":  # linear: the plain operator on the frame's rows (networkInNetwork.py:72-81)
            out = input.features.new_empty((0, self.nOut))
            SCN.NetworkInNetwork_updateOutput(input.features, out, self.weight, optionalTensor(self, 'bias'))
            output.features = out
        elif kind is None:
            out = input.features.new_empty((0, self.nOut))
            sparseconvnet.forward_pass_multiplyAdd_count += SCN.NetworkInNetwork_updateOutput(
                input.features, out, self.weight, optionalTensor(self, 'bias'))
            sparseconvnet.forward_pass_hidden_states += out.nelement()
            output.features = self._state.adopt(out)
        else:
            d = input.dirty
            n = input.features.size(0)
            out = self._state.grow(n, keep=min(n, self._state.buf.size(0)))
            rows, count = d.rows(d.scale.order.t)
            SCN.conv_rows(input.features, out, self.weight, SCN._opt(optionalTensor(self, 'bias')), None, 1,
                          rows, count, d.n_upper)
            output.features = out
            output.dirty = d
        return output

    def __repr__(self):
        return 'NetworkInNetwork' + str(self.nIn) + '->' + str(self.nOut)

    def input_spatial_size(self, out_size):
        return out_size
