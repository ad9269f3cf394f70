"""MaxPooling / AveragePooling / UnPooling, size 2 / stride 2 (reference:
sparseconvnet/maxPooling.py:71-105, averagePooling.py:13-66, unPooling.py:63-84), and
SparseToDense (sparseToDense.py:59-78).  Inference only; they are not part of the incremental
path (the reference has no Incre_* variant of them), so an incremental forward is refused."""
from torch.nn import Module

from . import SCN
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import toLongTensor


class _Pool(Module):
    _fn = None
    _name = ""

    def __init__(self, dimension, pool_size, pool_stride, nFeaturesToDrop=0):
        Module.__init__(self)
        self.dimension = dimension
        self.pool_size = toLongTensor(dimension, pool_size)
        self.pool_stride = toLongTensor(dimension, pool_stride)
        self.nFeaturesToDrop = nFeaturesToDrop

    def forward(self, input, increment=False):
        if increment:
            raise NotImplementedError("%s has no incremental forward" % self._name)
        output = SparseConvNetTensor(None, input.metadata, None)
        output.spatial_size = (input.spatial_size - self.pool_size) // self.pool_stride + 1
        assert ((output.spatial_size - 1) * self.pool_stride + self.pool_size == input.spatial_size).all()
        out = input.features.new_empty((0, 0))
        type(self)._fn(input.spatial_size, output.spatial_size, self.pool_size, self.pool_stride, input.metadata,
                       input.features, out, self.nFeaturesToDrop)
        output.features = out
        return output

    def input_spatial_size(self, out_size):
        return (out_size - 1) * self.pool_stride + self.pool_size

    def __repr__(self):
        s = self._name
        if self.pool_size.max().item() == self.pool_size.min().item() and \
                self.pool_stride.max().item() == self.pool_stride.min().item():
            s = s + str(self.pool_size[0].item()) + '/' + str(self.pool_stride[0].item())
        else:
            s = s + '(' + ','.join(str(i.item()) for i in self.pool_size) + ')/(' + \
                ','.join(str(i.item()) for i in self.pool_stride) + ')'
        if self.nFeaturesToDrop > 0:
            s = s + ' nFeaturesToDrop = ' + str(self.nFeaturesToDrop)
        return s


class MaxPooling(_Pool):
    _fn = staticmethod(SCN.MaxPooling_updateOutput)
    _name = "MaxPooling"


class AveragePooling(_Pool):
    _fn = staticmethod(SCN.AveragePooling_updateOutput)
    _name = "AveragePooling"


class UnPooling(Module):
    def __init__(self, dimension, pool_size, pool_stride, nFeaturesToDrop=0):
        Module.__init__(self)
        self.dimension = dimension
        self.pool_size = toLongTensor(dimension, pool_size)
        self.pool_stride = toLongTensor(dimension, pool_stride)
        self.nFeaturesToDrop = nFeaturesToDrop

    def forward(self, input, increment=False):
        if increment:
            raise NotImplementedError("UnPooling has no incremental forward")
        output = SparseConvNetTensor(None, input.metadata, None)
        output.spatial_size = (input.spatial_size - 1) * self.pool_stride + self.pool_size
        out = input.features.new_empty((0, 0))
        SCN.UnPooling_updateOutput(input.spatial_size, output.spatial_size, self.pool_size, self.pool_stride,
                                   input.metadata, input.features, out, self.nFeaturesToDrop)
        output.features = out
        return output

    def input_spatial_size(self, out_size):
        return (out_size - self.pool_size) // self.pool_stride + 1

    def __repr__(self):
        return 'UnPooling' + str(self.pool_size[0].item()) + '/' + str(self.pool_stride[0].item())


class SparseToDense(Module):
    """SparseConvNetTensor -> dense float tensor [batch, nPlanes, X, Y, Z] (zeros where no site is
    active), e.g. in front of dense torch layers."""

    def __init__(self, dimension, nPlanes):
        Module.__init__(self)
        self.dimension = dimension
        self.nPlanes = nPlanes

    def forward(self, input, increment=False):
        if increment:
            raise NotImplementedError("SparseToDense has no incremental forward")
        out = input.features.new_empty((0,))
        SCN.SparseToDense_updateOutput(input.spatial_size, input.metadata, input.features, out, self.nPlanes)
        return out

    def input_spatial_size(self, out_size):
        return out_size

    def __repr__(self):
        return 'SparseToDense(' + str(self.dimension) + ',' + str(self.nPlanes) + ')'
