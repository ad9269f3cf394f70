"""Deconvolution (reference: sparseconvnet/deconvolution.py:13-70); size 2 / stride 2 only."""
import torch
from torch.nn import Module, Parameter

import sparseconvnet

from . import SCN, incremental
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf, optionalTensor, toLongTensor


class Deconvolution(Module):
    def __init__(self, dimension, nIn, nOut, filter_size, filter_stride, bias):
        Module.__init__(self)
        self.dimension = dimension
        self.nIn = nIn
        self.nOut = nOut
        self.filter_size = toLongTensor(dimension, filter_size)
        self.filter_volume = self.filter_size.prod().item()
        self.filter_stride = toLongTensor(dimension, filter_stride)
        std = (2.0 / nIn / self.filter_volume) ** 0.5
        self.weight = Parameter(torch.Tensor(self.filter_volume, nIn, nOut).normal_(0, std))
        if bias:
            self.bias = Parameter(torch.Tensor(nOut).zero_())
        self._state = StateBuf()

    def forward(self, input, increment=False):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nIn
        output = SparseConvNetTensor(None, input.metadata, None)
        output.spatial_size = (input.spatial_size - 1) * self.filter_stride + self.filter_size
        kind = incremental.kind(increment)
        if kind == "residual":
            out = input.features.new_empty((0, self.nOut))
            SCN.Incre_Deconvolution_updateOutput(
                input.spatial_size, output.spatial_size, self.filter_size, self.filter_stride, input.metadata,
                input.features, out, self.weight, optionalTensor(self, 'bias'), self.save_meta,
                self.save_input_feats)
            output.features = out
        elif kind is None:
            out = input.features.new_empty((0, self.nOut))
            sparseconvnet.forward_pass_multiplyAdd_count += SCN.Deconvolution_updateOutput(
                input.spatial_size, output.spatial_size, self.filter_size, self.filter_stride, input.metadata,
                input.features, out, self.weight, optionalTensor(self, 'bias'))
            sparseconvnet.forward_pass_hidden_states += out.nelement()
            output.features = self._state.adopt(out)
            self.save_meta = output.metadata
            self.save_input_feats = input.features
        else:
            SCN._check_down(self.filter_size, self.filter_stride)
            m = input.metadata
            fine, coarse, down = m.down_rulebook(output.spatial_size, input.spatial_size)
            d = incremental.children(input.dirty, fine, down)
            out = self._state.grow(fine.n, keep=min(fine.n, self._state.buf.size(0)))
            rows, count = d.rows(m.deconv_order(fine, down), tag="by_offset")
            SCN.deconv_rows(input.features, out, self.weight, SCN._opt(optionalTensor(self, 'bias')),
                            down.parent.t, down.offset.t, rows, count, d.n_upper)
            output.features = out
            output.dirty = d
            self.save_input_feats = input.features
        return output

    def __repr__(self):
        s = 'Deconvolution ' + str(self.nIn) + '->' + str(self.nOut) + ' C'
        s += str(self.filter_size[0].item()) + '/' + str(self.filter_stride[0].item())
        return s

    def input_spatial_size(self, out_size):
        return (out_size - self.filter_size) // self.filter_stride + 1
