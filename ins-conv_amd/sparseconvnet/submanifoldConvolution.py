"""SubmanifoldConvolution (reference: sparseconvnet/submanifoldConvolution.py:18-83)."""
import torch
from torch.nn import Module, Parameter

import sparseconvnet

from . import SCN, incremental
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf, optionalTensor, toLongTensor


class SubmanifoldConvolution(Module):
    def __init__(self, dimension, nIn, nOut, filter_size, bias, dilated_rate=1):
        Module.__init__(self)
        self.dimension = dimension
        self.nIn = nIn
        self.nOut = nOut
        self.filter_size = toLongTensor(dimension, filter_size)
        self.filter_volume = self.filter_size.prod().item()
        std = (2.0 / nIn / self.filter_volume) ** 0.5
        self.weight = Parameter(torch.Tensor(self.filter_volume, nIn, nOut).normal_(0, std))
        self.dilated_rate = dilated_rate
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())
        self._state = StateBuf()

    def forward(self, input, increment=False):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn, (self.nIn, self.nOut, input)
        output = SparseConvNetTensor(None, input.metadata, input.spatial_size)
        kind = incremental.kind(increment)
        if kind == "residual":
            out = input.features.new_empty((0, self.nOut))
            SCN.Incre_SubmanifoldConvolution_updateOutput(
                input.spatial_size, self.filter_size, input.metadata, input.features, out, self.weight,
                optionalTensor(self, 'bias'), self.save_meta, self.save_input_feats, count_muladds=False)
            output.features = out
        elif kind is None:
            out = input.features.new_empty((0, self.nOut))
            sparseconvnet.forward_pass_multiplyAdd_count += SCN.SubmanifoldConvolution_updateOutput(
                input.spatial_size, self.filter_size, input.metadata, input.features, out, self.weight,
                optionalTensor(self, 'bias'), self.dilated_rate)
            sparseconvnet.forward_pass_hidden_states += out.nelement()
            output.features = self._state.adopt(out)
            self.save_meta = output.metadata
            self.save_input_feats = input.features
        else:
            m = input.metadata
            sc = m.ssc_rulebook(input.spatial_size)
            d = incremental.dilate(input.dirty)
            out = self._state.grow(sc.n, keep=min(sc.n, self._state.buf.size(0)))
            rows, count = d.rows(sc.order.t)
            SCN.conv_rows(input.features, out, self.weight, SCN._opt(optionalTensor(self, 'bias')), sc.nbr.t,
                          27, rows, count, d.n_upper)
            output.features = out
            output.dirty = d
            self.save_input_feats = input.features
        return output

    def __repr__(self):
        s = 'SubmanifoldConvolution ' + str(self.nIn) + '->' + str(self.nOut) + ' C'
        if self.filter_size.max() == self.filter_size.min():
            s = s + str(self.filter_size[0].item())
        else:
            s = s + '(' + ','.join(str(i.item()) for i in self.filter_size) + ')'
        return s

    def input_spatial_size(self, out_size):
        return out_size


class ValidConvolution(SubmanifoldConvolution):
    pass
