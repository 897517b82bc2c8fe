"""InputBatch: a SparseConvNetTensor filled point by point (reference:
sparseconvnet/inputBatch.py:13-127 over Metadata::setInputSpatialLocation(s), batchAddSample,
addSampleFromThresholdedTensor and generateRuleBooks2s2 / 3s2, Metadata/Metadata.cpp:74-147,
296-411).

The reference inserts every point into a host hash map as it arrives and grows a CPU feature
tensor row by row.  Here the calls only collect what they are given, on the host and in call
order; the first time somebody looks at `features` or `metadata` (a network's first module
does) the whole collection goes to the GPU once and the library builds the input level from
it in one pass, with the reference's outcome: a site's row is the rank of its first point, and
it holds that point's vector unless later points of the site came with overwrite=True, then
the last of those.  Setting more points afterwards rebuilds on the next look."""
import torch

from .metadata import Metadata
from .tensor import SparseConvNetTensor
from .utils import toLongTensor


class InputBatch(SparseConvNetTensor):
    def __init__(self, dimension, spatial_size):
        self.dimension = dimension
        self._coords = []     # int64 [k, dimension + 1] per call: coordinates, sample
        self._vectors = []    # float32 [k, planes] per call
        self._overwrite = []  # (k, overwrite) per call
        self._samples = 0     # samples added so far; the current one is the last
        self._current = -1
        self._dirty = False
        self._built = False
        self._features = torch.empty(0)
        self._metadata = Metadata(dimension)
        SparseConvNetTensor.__init__(self, self._features, self._metadata, toLongTensor(dimension, spatial_size))

    # ---- what the modules read ---------------------------------------------------------
    @property
    def features(self):
        self._build()
        return self._features

    @features.setter
    def features(self, value):  # .cuda() / .to() / .type() of the base class assign here
        self._features = value

    @property
    def metadata(self):
        self._build()
        return self._metadata

    @metadata.setter
    def metadata(self, value):
        self._metadata = value

    def cuda(self):
        return self  # the features are built on the GPU

    def to(self, device):
        if torch.device(device).type != "cuda":
            raise RuntimeError("an InputBatch of this library lives on the GPU")
        return self

    def _build(self):
        if not self._dirty:
            return
        self._dirty = False
        planes = {v.size(1) for v in self._vectors}
        if len(planes) > 1:
            raise ValueError("every vector of an InputBatch must have the same number of planes, got %s"
                             % sorted(planes))
        if self._built:
            self._metadata.clear()
        self._built = True
        n_planes = planes.pop() if planes else 0
        coords = torch.cat(self._coords) if self._coords else torch.zeros((0, self.dimension + 1),
                                                                          dtype=torch.int64)
        vectors = (torch.cat([v.to("cuda", non_blocking=True) for v in self._vectors]) if self._vectors
                   else torch.zeros((0, n_planes), dtype=torch.float32, device="cuda"))
        flags = None
        if any(o for _, o in self._overwrite):
            flags = torch.cat([torch.full((k,), 1 if o else 0, dtype=torch.uint8) for k, o in self._overwrite])
        self._features = self._metadata.inputBatch(self.spatial_size, coords, vectors, flags, self._samples)

    # ---- filling -----------------------------------------------------------------------
    def add_sample(self):
        self._samples += 1
        self._current = self._samples - 1
        self._dirty = True

    def _append(self, coords, vectors, overwrite):
        self._coords.append(coords)
        self._vectors.append(vectors)
        self._overwrite.append((coords.size(0), bool(overwrite)))
        self._dirty = True

    def _check_inside(self, l):
        assert l.numel() == 0 or (l.min() >= 0 and (self.spatial_size.expand_as(l) - l).min() > 0), \
            "location outside the spatial size"

    def set_location(self, location, vector, overwrite=False):
        location = location.detach().cpu().long().reshape(1, -1)
        self._check_inside(location)
        self.set_locations_(location, vector.reshape(1, -1), overwrite)

    def set_location_(self, location, vector, overwrite=False):
        self.set_locations_(location.detach().cpu().long().reshape(1, -1), vector.reshape(1, -1), overwrite)

    def set_locations(self, locations, vectors, overwrite=False):
        """locations: LongTensor [n, dimension] (points of the current sample) or
        [n, dimension + 1] (last column: the sample, 0-based; the batch grows as needed);
        vectors: FloatTensor [n, planes]."""
        locations = locations.detach().cpu().long()
        self._check_inside(locations[:, :self.dimension])
        self.set_locations_(locations, vectors, overwrite)

    def set_locations_(self, locations, vectors, overwrite=False):
        locations = locations.detach().cpu().long()
        vectors = vectors.detach().float()
        assert locations.dim() == 2 and vectors.dim() == 2 and locations.size(0) == vectors.size(0), \
            (locations.shape, vectors.shape)
        if locations.size(1) == self.dimension:
            if self._current < 0:
                raise RuntimeError("call add_sample() first, please")
            sample = torch.full((locations.size(0), 1), self._current, dtype=torch.int64)
            locations = torch.cat([locations, sample], 1)
        elif locations.size(1) == self.dimension + 1:
            if locations.size(0):
                assert locations[:, -1].min() >= 0, "negative sample index"
                self._samples = max(self._samples, int(locations[:, -1].max()) + 1)
        else:
            raise ValueError("locations must have %d or %d columns" % (self.dimension, self.dimension + 1))
        self._append(locations.contiguous(), vectors.contiguous(), overwrite)

    def add_sample_from_tensor(self, tensor, offset, threshold=0):
        """A new sample from a dense tensor [size_1, .., size_d, planes] placed at `offset`:
        cells with a plane above `threshold` in magnitude, inside the spatial size, become
        points, visited with the last dimension fastest."""
        tensor = tensor.detach().float()
        assert tensor.dim() == self.dimension + 1
        offset = toLongTensor(self.dimension, offset)
        self._samples += 1
        cells = (tensor.abs() > threshold).any(-1).nonzero()
        where = cells.cpu() + offset
        inside = ((where >= 0) & (where < self.spatial_size)).all(1)
        cells, where = cells[inside.to(cells.device)], where[inside]
        vectors = tensor[tuple(cells.t())] if cells.numel() else tensor.new_zeros((0, tensor.size(-1)))
        sample = torch.full((where.size(0), 1), self._samples - 1, dtype=torch.int64)
        self._append(torch.cat([where, sample], 1).contiguous(), vectors.contiguous(), False)

    def precompute_metadata(self, size):
        """Optional: builds the rulebooks of every level ahead of the network (3^d submanifold
        plus size-2 or size-3 stride-2), on the library's construction stream."""
        if size == 2:
            self.metadata.generateRuleBooks2s2()
        if size == 3:
            self.metadata.generateRuleBooks3s2()

    # Deprecated method names of the reference.
    addSample = add_sample
    setLocation = set_location
    setLocation_ = set_location_
    setLocations = set_locations
    setLocations_ = set_locations_
    addSampleFromTensor = add_sample_from_tensor
    precomputeMetadata = precompute_metadata
