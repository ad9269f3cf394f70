"""SparseConvNetTensor: a feature matrix, the Metadata that says which sites its rows belong to,
and the spatial size of the scale (reference: sparseconvnet/sparseConvNetTensor.py).

`dirty` is an addition: during an exact incremental forward it names the rows of `features`
that changed in this frame (None otherwise).
"""


class SparseConvNetTensor(object):
    def __init__(self, features=None, metadata=None, spatial_size=None):
        self.features, self.metadata, self.spatial_size = features, metadata, spatial_size
        self.dirty = None

    def _with_features(self, fn):
        self.features = fn(self.features)
        return self

    # torch.Tensor-like movers; each works in place on `features` and returns self
    def to(self, device):
        return self._with_features(lambda f: f.to(device))

    def cuda(self):
        return self._with_features(lambda f: f.cuda())

    def cpu(self):
        return self._with_features(lambda f: f.cpu())

    def type(self, t=None):
        if not t:
            return self.features.type()
        return self._with_features(lambda f: f.type(t))

    def detach(self):
        out = SparseConvNetTensor(self.features.detach(), self.metadata, self.spatial_size)
        out.dirty = self.dirty
        return out

    def get_spatial_locations(self, spatial_size=None):
        """Long [N,4] (x, y, z, batch index) of the active sites, rows in feature order."""
        size = self.spatial_size if spatial_size is None else spatial_size
        return self.metadata.getSpatialLocations(size)

    def __repr__(self):
        where = self.get_spatial_locations() if self.metadata else None
        return "SparseConvNetTensor<<features=%r,features.shape=%r,batch_locations=%r,spatial size=%r>>" % (
            self.features, self.features.shape, where, self.spatial_size)
