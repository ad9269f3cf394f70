"""BatchNormalization (+ReLU / LeakyReLU), inference (reference: sparseconvnet/batchNormalization.py:13-110)."""
import torch
from torch.nn import Module, Parameter

from . import SCN, incremental
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf, optionalTensor


class BatchNormalization(Module):
    """
    nPlanes : number of input planes; eps : stabilises the standard deviation;
    momentum : kept for state_dict compatibility (training is not provided);
    leakiness : 0 for ReLU, values in (0,1) for LeakyReLU, 1 for no activation.
    """

    def __init__(self, nPlanes, eps=1e-4, momentum=0.9, affine=True, leakiness=1):
        Module.__init__(self)
        self.nPlanes = nPlanes
        self.eps = eps
        self.momentum = momentum
        self.affine = affine
        self.leakiness = leakiness
        self.register_buffer("running_mean", torch.Tensor(nPlanes).fill_(0))
        self.register_buffer("running_var", torch.Tensor(nPlanes).fill_(1))
        if affine:
            self.weight = Parameter(torch.Tensor(nPlanes).fill_(1))
            self.bias = Parameter(torch.Tensor(nPlanes).fill_(0))
        self._state = StateBuf()

    def forward(self, input, increment=False):
        assert input.features.nelement() == 0 or input.features.size(1) == self.nPlanes, (
            self.nPlanes, input.features.shape)
        if self.training:
            raise NotImplementedError("training-mode batch norm is outside the inference path; call .eval()")
        output = SparseConvNetTensor(None, input.metadata, input.spatial_size)
        kind = incremental.kind(increment)
        if kind == "residual":
            out = input.features.new_empty((0, self.nPlanes))
            SCN.Incre_BatchNormalization_updateOutput(
                input.features, out, None, None, self.running_mean, self.running_var,
                optionalTensor(self, 'weight'), optionalTensor(self, 'bias'), self.eps, self.momentum, False,
                self.leakiness, output.metadata, self.save_output.metadata, self.save_output.features,
                self.save_input.features, input.spatial_size)
            output.features = out
            return output
        if kind is None:
            out = input.features.new_empty((0, self.nPlanes))
            SCN.BatchNormalization_updateOutput(
                input.features, out, None, None, self.running_mean, self.running_var,
                optionalTensor(self, 'weight'), optionalTensor(self, 'bias'), self.eps, self.momentum, False,
                self.leakiness)
            output.features = self._state.adopt(out)
        else:
            d = input.dirty
            n = input.features.size(0)
            out = self._state.grow(n, keep=min(n, self._state.buf.size(0)))
            rows, count = d.rows(d.scale.order.t)
            SCN.bn_rows(input.features, out, self.running_mean, self.running_var,
                        SCN._opt(optionalTensor(self, 'weight')), SCN._opt(optionalTensor(self, 'bias')),
                        float(self.eps), float(self.leakiness), rows, count, d.n_upper)
            output.features = out
            output.dirty = d
        self.save_output = output
        self.save_input = input
        return output

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        s = 'BatchNorm(' + str(self.nPlanes) + ',eps=' + str(self.eps) + ',momentum=' + str(self.momentum) + \
            ',affine=' + str(self.affine)
        if self.leakiness > 0:
            s = s + ',leakiness=' + str(self.leakiness)
        return s + ')'


class BatchNormReLU(BatchNormalization):
    def __init__(self, nPlanes, eps=1e-4, momentum=0.9):
        BatchNormalization.__init__(self, nPlanes, eps, momentum, True, 0)


class BatchNormLeakyReLU(BatchNormalization):
    def __init__(self, nPlanes, eps=1e-4, momentum=0.9, leakiness=0.333):
        BatchNormalization.__init__(self, nPlanes, eps, momentum, True, leakiness)
