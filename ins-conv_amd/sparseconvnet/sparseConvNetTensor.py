"""SparseConvNetTensor (reference: sparseconvnet/sparseConvNetTensor.py).

`dirty` is an addition: during an incremental forward it names the rows of `features` that
changed in this frame (None during a full forward).
"""


class SparseConvNetTensor(object):
    def __init__(self, features=None, metadata=None, spatial_size=None):
        self.features = features
        self.metadata = metadata
        self.spatial_size = spatial_size
        self.dirty = None

    def get_spatial_locations(self, spatial_size=None):
        "Coordinates and batch index for the active spatial locations"
        if spatial_size is None:
            spatial_size = self.spatial_size
        return self.metadata.getSpatialLocations(spatial_size)

    def to(self, device):
        self.features = self.features.to(device)
        return self

    def type(self, t=None):
        if t:
            self.features = self.features.type(t)
            return self
        return self.features.type()

    def cuda(self):
        self.features = self.features.cuda()
        return self

    def cpu(self):
        self.features = self.features.cpu()
        return self

    def detach(self):
        x = SparseConvNetTensor(self.features.detach(), self.metadata, self.spatial_size)
        x.dirty = self.dirty
        return x

    def __repr__(self):
        sl = self.get_spatial_locations() if self.metadata else None
        return ('SparseConvNetTensor<<features=' + repr(self.features) + ',features.shape=' +
                repr(self.features.shape) + ',batch_locations=' + repr(sl) + ',spatial size=' +
                repr(self.spatial_size) + '>>')
