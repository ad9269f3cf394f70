"""InputLayer / OutputLayer (reference: sparseconvnet/ioLayers.py:15-119,324-376)."""
import ctypes

import torch
from torch.nn import Module

from . import SCN, incremental
from ._lib import lib, ptr, stream_ptr
from .metadata import Metadata
from .sparseConvNetTensor import SparseConvNetTensor
from .utils import StateBuf, toLongTensor

I64 = ctypes.c_int64


class InputLayer(Module):
    """
    Takes a tuple (coords, features, batch_size [optional])
    * coords is 2d torch.LongTensor with size N x dimension (batch size == 1) or
      N x (dimension+1) (last column is the batch index)
    * features is a CUDA float tensor with size N x n_feature_planes
    mode == 0 input guaranteed to have no duplicates, 1 keep the first item at each location,
    2 keep the last, 3 sum, 4 average (1 and 2 as implemented by the reference's rule
    builder, Metadata/IOLayersRules.h:104-115).

    forward(input, increment=True) appends the given points to the sites of the last full
    forward and marks the touched sites dirty; the output then holds the features of ALL
    sites, with only the dirty rows recomputed downstream.  With increment="residual" (or
    incremental.set_mode("residual")) the frame is processed the reference's way instead: a
    site set of its own, features as differences to the saved state.
    """

    def __init__(self, dimension, spatial_size, mode=3, normal_guide_scale=10240):
        Module.__init__(self)
        self.dimension = dimension
        self.spatial_size = toLongTensor(dimension, spatial_size)
        self.mode = mode
        self.normal_guide_scale = normal_guide_scale
        self.device = None
        self._state = StateBuf()

    def to(self, device):
        self.device = device
        return self

    def forward(self, input, increment=False):
        assert len(input) >= 2, len(input)
        coords, feats = input[0], input[1]
        batch_size = input[2] if len(input) > 2 else 0
        kind = incremental.kind(increment)
        if kind == "residual":
            # the frame gets a site set of its own; the saved output stays as it is (ioLayers.py:70-80)
            prev = self.save_output
            output = SparseConvNetTensor(metadata=Metadata(self.dimension), spatial_size=self.spatial_size)
            output.metadata._bind(feats.device)
            out = feats.new_empty((0, feats.size(1)))
            SCN.Incre_InputLayer_updateOutput(output.metadata, self.spatial_size, coords, feats, out, batch_size,
                                              self.mode, prev.metadata, prev.features)
            output.features = out
            return output
        if kind is None:
            output = SparseConvNetTensor(metadata=Metadata(self.dimension), spatial_size=self.spatial_size)
            m = output.metadata
            m._bind(feats.device)
            out = feats.new_empty((0, feats.size(1)))
            SCN.InputLayer_updateOutput(m, self.spatial_size, coords, feats, out, batch_size, self.mode)
            output.features = self._state.adopt(out)
            self.save_output = output
            return output
        # incremental: extend the saved site set
        if self.mode in (1, 2):
            raise NotImplementedError("incremental input needs mode 0, 3 or 4")
        prev = self.save_output
        m = prev.metadata
        sc = m.scale(self.spatial_size)
        n_before = sc.n
        C = feats.size(1)
        sop, _ = SCN._append_points(m, sc, coords, feats)
        d = incremental.from_points(sc, sop)
        m.ssc_rulebook(self.spatial_size)  # neighbour map / order for the new sites
        out = self._state.grow(sc.n, keep=n_before)
        rows, count = d.rows(sc.order.t)
        lib.insc_input_finish(ptr(m.in_sum.t), ptr(m.in_cnt.t), int(self.mode), ptr(out), I64(C), ptr(rows),
                              ptr(count), I64(d.n_upper), int(C), stream_ptr())
        output = SparseConvNetTensor(out, m, self.spatial_size)
        output.dirty = d
        self.save_output = output
        return output

    def input_spatial_size(self, out_size):
        return out_size


class OutputLayer(Module):
    """
    Takes a SparseConvNetTensor and returns a float tensor with one row per input row given
    to the InputLayer.  After an incremental forward the rows are those of the increment's
    points (as in the reference); set `all_points = True` to get a row for every point seen
    since the last full forward.
    """

    def __init__(self, dimension):
        Module.__init__(self)
        self.dimension = dimension
        self.all_points = False

    def forward(self, input, increment=False):
        m = input.metadata
        f = input.features
        if incremental.kind(increment) == "residual":
            out = f.new_empty((0, f.size(1)))
            SCN.Incre_OutputLayer_updateOutput(m, f, out, self.save_meta, self.save_input_feats)
            return out
        sop = m.site_of_all_points if (not increment or self.all_points) else m.site_of_point
        out = torch.empty((sop.numel(), f.size(1)), dtype=f.dtype, device=f.device)
        if sop.numel():
            lib.insc_output_gather(ptr(f), I64(SCN._ld(f)), ptr(sop), I64(sop.numel()), int(f.size(1)), ptr(out),
                                   stream_ptr())
        self.save_input_feats = f
        self.save_meta = m
        return out

    def input_spatial_size(self, out_size):
        return out_size
