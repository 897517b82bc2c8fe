"""SparseConvNetTensor: features [nActive, planes] + the Metadata that says where they
sit + the spatial size of the level (reference: sparseconvnet/sparseConvNetTensor.py:12-63)."""


class SparseConvNetTensor(object):
    def __init__(self, features=None, metadata=None, spatial_size=None):
        self.features = features
        self.metadata = metadata
        self.spatial_size = spatial_size

    def get_spatial_locations(self, spatial_size=None):
        "Coordinates and batch index for the active spatial locations"
        size = self.spatial_size if spatial_size is None else spatial_size
        return self.metadata.getSpatialLocations(size)

    def batch_size(self):
        return self.metadata.getBatchSize(self.spatial_size)

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
        return SparseConvNetTensor(self.features.detach(), self.metadata, self.spatial_size)

    @property
    def requires_grad(self):
        return self.features.requires_grad

    def __repr__(self):
        loc = self.get_spatial_locations() if self.metadata else None
        return ('SparseConvNetTensor<<features=' + repr(self.features) + ',features.shape=' +
                repr(self.features.shape) + ',batch_locations=' + repr(loc) + ',batch_locations.shape=' +
                repr(loc.shape if self.metadata else None) + ',spatial size=' + repr(self.spatial_size) + '>>')
