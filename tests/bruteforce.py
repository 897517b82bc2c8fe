"""Independent statements of what each part of the path computes: dictionaries
and loops on small inputs, and dense torch routines.  Nothing here shares code
with oracle/ or with the library; the tests pin both against these."""
import itertools

import numpy as np
import torch
import torch.nn.functional as F


def filter_offsets(dim, size):
    """Filter taps in rulebook order: row-major over the box, last dimension fastest."""
    size = np.broadcast_to(np.asarray(size), (dim,))
    return list(itertools.product(*[range(int(s)) for s in size]))


def first_occurrence_rows(coords):
    """Row id of every input point = rank of its (coords, batch) among first occurrences."""
    seen = {}
    row_of = np.zeros(len(coords), np.int64)
    for i, c in enumerate(map(tuple, coords)):
        if c not in seen:
            seen[c] = len(seen)
        row_of[i] = seen[c]
    return row_of, len(seen)


def input_layer_values(coords, feats, mode):
    """Features after the input layer for modes 1 (first), 2 (last), 3 (sum), 4 (mean)."""
    row_of, n = first_occurrence_rows(coords)
    out = np.zeros((n, feats.shape[1]), np.float64)
    cnt = np.bincount(row_of, minlength=n)
    if mode == 1:
        for i in range(len(coords) - 1, -1, -1):
            out[row_of[i]] = feats[i]
    elif mode == 2:
        for i in range(len(coords)):
            out[row_of[i]] = feats[i]
    else:
        np.add.at(out, row_of, feats.astype(np.float64))
        if mode == 4:
            out /= cnt[:, None]
    return out.astype(np.float32), row_of


def bl_groups(coords):
    """Batch-by-length input [B, L, d]: the flat input indices of every output row, rows in
    first-occurrence order sample after sample, positions with a negative first coordinate
    skipped; plus the (coords, sample) location of every row."""
    B, L, d = coords.shape
    groups, loc = [], []
    for b in range(B):
        seen = {}
        for l in range(L):
            c = tuple(int(v) for v in coords[b, l])
            if c[0] < 0:
                continue
            if c not in seen:
                seen[c] = len(groups)
                groups.append([])
                loc.append(c + (b,))
            groups[seen[c]].append(b * L + l)
    return groups, np.asarray(loc, np.int64).reshape(len(loc), d + 1)


class PointTable:
    """The point-at-a-time input as a dictionary: a new (coordinates, sample) takes the next
    row and the vector; a known one keeps its vector unless the point overwrites."""

    def __init__(self):
        self.rows = {}
        self.vectors = []

    def set(self, key, vector, overwrite):
        key = tuple(int(v) for v in key)
        if key not in self.rows:
            self.rows[key] = len(self.rows)
            self.vectors.append(np.array(vector, np.float32))
        elif overwrite:
            self.vectors[self.rows[key]] = np.array(vector, np.float32)

    def dense_block(self, tensor, offset, spatial, sample, threshold):
        """Cells of a dense [size..., planes] block at `offset` with some |plane| > threshold,
        inside the grid, in row-major order, as points of a new sample."""
        spatial = np.broadcast_to(np.asarray(spatial), (tensor.ndim - 1,))
        for cell in itertools.product(*[range(n) for n in tensor.shape[:-1]]):
            where = [c + int(o) for c, o in zip(cell, offset)]
            if not (np.abs(tensor[cell]) > threshold).any():
                continue
            if any(w < 0 or w >= int(s) for w, s in zip(where, spatial)):
                continue
            self.set(tuple(where) + (sample,), tensor[cell], False)

    def locations(self):
        return np.array(sorted(self.rows, key=self.rows.get), np.int64).reshape(len(self.rows), -1)

    def features(self):
        return np.array(self.vectors, np.float32)


def submanifold_triples(loc, dim, size):
    """Set of (k, in_site, out_site) as coordinate tuples: in = out + tap - size//2, same sample."""
    size = np.broadcast_to(np.asarray(size), (dim,))
    sites = set(map(tuple, loc))
    out = set()
    for j in sites:
        for k, tap in enumerate(filter_offsets(dim, size)):
            i = tuple(j[d] + tap[d] - int(size[d]) // 2 for d in range(dim)) + (j[dim],)
            if i in sites:
                out.add((k,) + i + j)
    return out


def strided_triples(loc, dim, size, stride, out_size):
    """Set of (k, in_site, out_site): out*stride + tap = in, 0 <= out < out_size."""
    size = np.broadcast_to(np.asarray(size), (dim,))
    stride = np.broadcast_to(np.asarray(stride), (dim,))
    out_size = np.broadcast_to(np.asarray(out_size), (dim,))
    res = set()
    for p in map(tuple, loc):
        for k, tap in enumerate(filter_offsets(dim, size)):
            ok = True
            j = []
            for d in range(dim):
                q = p[d] - tap[d]
                if q < 0 or q % int(stride[d]) or q // int(stride[d]) >= int(out_size[d]):
                    ok = False
                    break
                j.append(q // int(stride[d]))
            if ok:
                res.add((k,) + p + tuple(j) + (p[dim],))
    return res


def triples_of(canon):
    return set(map(tuple, canon.tolist()))


def to_dense(loc, feats, spatial, batch):
    """[B, C, spatial...] tensor with zeros at inactive sites."""
    dim = loc.shape[1] - 1
    spatial = [int(s) for s in np.broadcast_to(np.asarray(spatial), (dim,))]
    d = torch.zeros([batch, feats.shape[1]] + spatial, dtype=torch.float64)
    idx = (torch.as_tensor(loc[:, -1]), slice(None)) + tuple(
        torch.as_tensor(loc[:, i]) for i in range(dim))
    d[idx] = torch.as_tensor(feats, dtype=torch.float64)
    return d


def sample_dense(dense, loc):
    dim = loc.shape[1] - 1
    idx = (torch.as_tensor(loc[:, -1]), slice(None)) + tuple(
        torch.as_tensor(loc[:, i]) for i in range(dim))
    return dense[idx].numpy()


def dense_weight(w, dim, size):
    """[K, 1, nIn, nOut] -> torch conv weight [nOut, nIn, size...] (cross-correlation)."""
    size = [int(s) for s in np.broadcast_to(np.asarray(size), (dim,))]
    K, g, ci, co = w.shape
    assert g == 1
    return torch.as_tensor(w, dtype=torch.float64).reshape(size + [ci, co]).permute(
        dim + 1, dim, *range(dim)).contiguous()


_CONV = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}
_CONVT = {1: F.conv_transpose1d, 2: F.conv_transpose2d, 3: F.conv_transpose3d}
_AVG = {1: F.avg_pool1d, 2: F.avg_pool2d, 3: F.avg_pool3d}
_POOL = {1: F.max_pool1d, 2: F.max_pool2d, 3: F.max_pool3d}


def triple_conv(triples, loc_in, loc_out, feats, w, bias=None):
    """y[out] = bias + sum over (k, in, out) of x[in] @ w[k]; for dimensions torch has no
    dense convolution for."""
    dim = loc_in.shape[1] - 1
    row_in = {tuple(c): r for r, c in enumerate(loc_in.tolist())}
    row_out = {tuple(c): r for r, c in enumerate(loc_out.tolist())}
    y = np.zeros((len(loc_out), w.shape[3]), np.float64)
    if bias is not None:
        y += bias
    for t in triples:
        k, i, j = t[0], t[1:2 + dim], t[2 + dim:]
        y[row_out[j]] += feats[row_in[i]].astype(np.float64) @ w[k, 0].astype(np.float64)
    return y


def rule_rows(triples, loc_in, loc_out):
    """(k, in site, out site) triples as rows (k, in row, out row) of the two site lists."""
    dim = loc_in.shape[1] - 1
    row_in = {tuple(c): r for r, c in enumerate(loc_in.tolist())}
    row_out = {tuple(c): r for r, c in enumerate(loc_out.tolist())}
    return [(t[0], row_in[t[1:2 + dim]], row_out[t[2 + dim:]]) for t in triples]


def rows_strided_ops(rows, x, y, w, w2, n_in, n_out, K, bias=None):
    """Every op of a strided rulebook as loops over its rules, for dimensions beyond torch's
    dense routines: convolution, max pooling (from zero), average pooling, and from the coarse
    rows y back to the fine level unpooling and transposed convolution."""
    x64, y64 = x.astype(np.float64), y.astype(np.float64)
    conv = np.zeros((n_out, w.shape[3])) + (0 if bias is None else bias)
    mp = np.zeros((n_out, x.shape[1]))
    ap = np.zeros((n_out, x.shape[1]))
    up = np.zeros((n_in, y.shape[1]))
    dz = np.zeros((n_in, w2.shape[3]))
    for k, i, j in rows:
        conv[j] += x64[i] @ w[k, 0].astype(np.float64)
        mp[j] = np.maximum(mp[j], x64[i])
        ap[j] += x64[i] / K
        up[i] += y64[j]
        dz[i] += y64[j] @ w2[k, 0].astype(np.float64)
    return conv, mp, ap, up, dz


def dense_subm_conv(loc, feats, w, spatial, size, batch, bias=None):
    dim = loc.shape[1] - 1
    if dim not in _CONV:
        return triple_conv(submanifold_triples(loc, dim, size), loc, loc, feats, w, bias)
    sz = [int(s) for s in np.broadcast_to(np.asarray(size), (dim,))]
    x = to_dense(loc, feats, spatial, batch)
    b = None if bias is None else torch.as_tensor(bias, dtype=torch.float64)
    # padding size//2 on the low side, size-1-size//2 on the high side
    pads = []
    for s in reversed(sz):
        pads += [s // 2, s - 1 - s // 2]
    y = _CONV[dim](F.pad(x, pads), dense_weight(w, dim, sz), b)
    return sample_dense(y, loc)


def dense_strided_conv(loc, feats, w, spatial, size, stride, batch, bias=None):
    dim = loc.shape[1] - 1
    x = to_dense(loc, feats, spatial, batch)
    st = [int(s) for s in np.broadcast_to(np.asarray(stride), (dim,))]
    b = None if bias is None else torch.as_tensor(bias, dtype=torch.float64)
    return _CONV[dim](x, dense_weight(w, dim, size), b, stride=st)


def dense_deconv(loc_coarse, feats, w, coarse_spatial, size, stride, batch):
    dim = loc_coarse.shape[1] - 1
    x = to_dense(loc_coarse, feats, coarse_spatial, batch)
    st = [int(s) for s in np.broadcast_to(np.asarray(stride), (dim,))]
    # conv_transpose weight is [in, out, size...]
    wd = dense_weight(w, dim, size).transpose(0, 1).contiguous()
    return _CONVT[dim](x, wd, stride=st)


def dense_maxpool(loc, feats, spatial, size, stride, batch):
    dim = loc.shape[1] - 1
    x = to_dense(loc, feats, spatial, batch)
    sz = [int(s) for s in np.broadcast_to(np.asarray(size), (dim,))]
    st = [int(s) for s in np.broadcast_to(np.asarray(stride), (dim,))]
    # the output starts at zero and only grows (CPU/MaxPooling.cpp:17-18,50): a window whose
    # sites are all active and negative still yields 0
    return _POOL[dim](x, sz, st).clamp(min=0)


def dense_avgpool(loc, feats, spatial, size, stride, batch):
    """Sum of the window over its volume, absent sites as zeros (CPU/AveragePooling.cpp:19,59)."""
    dim = loc.shape[1] - 1
    x = to_dense(loc, feats, spatial, batch)
    sz = [int(s) for s in np.broadcast_to(np.asarray(size), (dim,))]
    st = [int(s) for s in np.broadcast_to(np.asarray(stride), (dim,))]
    return _AVG[dim](x, sz, st)


def active_mask(loc, spatial, batch):
    return to_dense(loc, np.ones((len(loc), 1)), spatial, batch) > 0


def random_sites(rng, dim, spatial, n, batch, duplicates=0):
    pts = rng.integers(0, spatial, (n, dim))
    b = rng.integers(0, batch, (n, 1))
    c = np.concatenate([pts, b], 1).astype(np.int64)
    if duplicates:
        c = np.concatenate([c, c[rng.integers(0, n, duplicates)]], 0)
        c = c[rng.permutation(len(c))]
    return c
