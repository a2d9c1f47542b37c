"""Numpy restatement of the reference's octree build and neighbour search.

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this file.

Every function names the reference lines it follows (paths relative to the
reference checkout).  All integer results are int64/int32 exactly as the
reference produces them.
"""

import numpy as np

I64 = np.int64


# --------------------------------------------------------------------------
# Morton ("shuffled") keys        ocnn/octree/shuffled_key.py:12-115
# --------------------------------------------------------------------------

def _spread(v, nbits, shift):
  """Bit i of v goes to bit 3*i + shift (shuffled_key.py:37-44)."""
  v = v.astype(I64)
  out = np.zeros_like(v)
  for i in range(nbits):
    out |= ((v >> i) & 1) << (3 * i + shift)
  return out


def _to_long(v):
  """``Tensor.long()``: floats truncate toward zero, integers pass through."""
  v = np.asarray(v)
  if np.issubdtype(v.dtype, np.floating):
    v = np.trunc(v)
  return v.astype(I64)


def xyz2key(x, y, z, b=None, depth=16):
  """shuffled_key.py:60-90.  x/y/z are truncated to int64 first (``.long()``),
  masked to 8 bits (or ``depth`` bits when depth <= 8), table-encoded, and for
  depth > 8 a second group from bits 8.. is placed at bit 24.  The batch index
  goes to bits >= 48."""
  x, y, z = _to_long(x), _to_long(y), _to_long(z)
  mask = 255 if depth > 8 else (1 << depth) - 1
  key = _spread(x & mask, 8, 2) | _spread(y & mask, 8, 1) | _spread(z & mask, 8, 0)
  if depth > 8:
    mask = (1 << (depth - 8)) - 1
    hi = (_spread((x >> 8) & mask, 8, 2) | _spread((y >> 8) & mask, 8, 1) |
          _spread((z >> 8) & mask, 8, 0))
    key = (hi << 24) | key
  if b is not None:
    bb = _to_long(b)
    key = (bb << 48) | key
  return key


def key2xyz(key, depth=16):
  """shuffled_key.py:93-115.  Decodes ceil(depth/3) groups of 9 key bits."""
  key = np.asarray(key).astype(I64)
  b = key >> 48
  key = key & ((1 << 48) - 1)
  n = (depth + 2) // 3
  x = np.zeros_like(key)
  y = np.zeros_like(key)
  z = np.zeros_like(key)
  for i in range(3 * n):
    x |= ((key >> (3 * i + 2)) & 1) << i
    y |= ((key >> (3 * i + 1)) & 1) << i
    z |= ((key >> (3 * i + 0)) & 1) << i
  return x, y, z, b


# --------------------------------------------------------------------------
# lookup tables                    ocnn/octree/octree.py:85-106, utils.py:46-74
# --------------------------------------------------------------------------

def range_grid(lo, hi):
  r = np.arange(lo, hi + 1, dtype=I64)
  g = np.stack(np.meshgrid(r, r, r, indexing='ij'), axis=-1)
  return g.reshape(-1, 3)


def neigh_luts():
  """octree.py:87-95: for child j (center in {2,3}^3) and slot k (disp in
  {-1,0,1}^3): which of the parent's 27 neighbours holds the cell, and which
  of that node's 8 children it is."""
  center = range_grid(2, 3)                       # (8, 3)
  disp = range_grid(-1, 1)                        # (27, 3)
  g = center[:, None, :] + disp[None, :, :]       # (8, 27, 3), values 1..4
  parent = g // 2                                 # values >= 0: trunc == floor
  child = g % 2
  lut_parent = (parent * np.array([9, 3, 1])).sum(-1)
  lut_child = (child * np.array([4, 2, 1])).sum(-1)
  return lut_parent.astype(I64), lut_child.astype(I64)


LUT_KERNEL = {                                    # octree.py:98-106
    '222': [13, 14, 16, 17, 22, 23, 25, 26],
    '311': [4, 13, 22],
    '131': [10, 13, 16],
    '113': [12, 13, 14],
    '331': [1, 4, 7, 10, 13, 16, 19, 22, 25],
    '313': [3, 4, 5, 12, 13, 14, 21, 22, 23],
    '133': [9, 10, 11, 12, 13, 14, 15, 16, 17],
}


# --------------------------------------------------------------------------
# octree container (plain dict-like object)
# --------------------------------------------------------------------------

class OctreeRef:
  """Holds what the reference's Octree holds after a build (octree.py:55-106)."""

  def __init__(self, depth, full_depth=2, batch_size=1):
    self.depth, self.full_depth, self.batch_size = depth, full_depth, batch_size
    n = depth + 1
    self.keys = [None] * n
    self.children = [None] * n
    self.neighs = [None] * n
    self.points = [None] * n
    self.normals = [None] * n
    self.features = [None] * n
    self.nnum = np.zeros(n, I64)
    self.nnum_nempty = np.zeros(n, I64)

  # octree.py:147-199 ------------------------------------------------------
  def nempty_mask(self, d):
    return self.children[d] >= 0

  def nempty_index(self, d):
    return np.nonzero(self.nempty_mask(d))[0].astype(I64)

  def remap_nempty_neigh(self, neigh, d):
    """octree.py:188-199: valid entries become the non-empty ordinal."""
    neigh = neigh.copy()
    valid = neigh >= 0
    neigh[valid] = self.children[d][neigh[valid]].astype(I64)
    return neigh

  def nempty_neigh(self, d):
    return self.remap_nempty_neigh(self.neighs[d][self.nempty_index(d)], d)

  # octree.py:490-523 ------------------------------------------------------
  def get_neigh(self, depth, kernel='333', stride=1, nempty=False):
    if stride == 1 and not nempty:
      neigh = self.neighs[depth]
    elif stride == 2 and not nempty:
      neigh = self.neighs[depth][::8].copy()
    elif stride == 1 and nempty:
      neigh = self.nempty_neigh(depth)
    elif stride == 2 and nempty:
      neigh = self.remap_nempty_neigh(self.neighs[depth][::8], depth)
    else:
      raise ValueError('Unsupported stride {}'.format(stride))
    if kernel == '333':
      return neigh
    if kernel in LUT_KERNEL:
      return neigh[:, LUT_KERNEL[kernel]]
    raise ValueError('Unsupported kernel {}'.format(kernel))

  # octree.py:525-568 ------------------------------------------------------
  def get_input_feature(self, feature, nempty=False):
    """N: leaf normals; D: displacement = <local point, normal>; L: local point = frac(p) - 0.5;
    P: point scaled to [-1, 1]; F: leaf features; all fp32, in this order; zero rows for the
    empty leaves unless nempty."""
    d = self.depth
    feature = feature.upper()
    parts = []
    pts = self.points[d].astype(np.float32)
    # torch's frac() is x - trunc(x); the leaf points are non-negative
    local = (pts - np.trunc(pts)).astype(np.float32) - np.float32(0.5)
    if 'N' in feature:
      parts.append(self.normals[d].astype(np.float32))
    if 'D' in feature:
      parts.append((local * self.normals[d].astype(np.float32)).sum(1, keepdims=True, dtype=np.float32))
    if 'L' in feature:
      parts.append(local)
    if 'P' in feature:
      parts.append(pts * np.float32(2.0 ** (1 - d)) - np.float32(1.0))
    if 'F' in feature:
      parts.append(self.features[d].astype(np.float32))
    out = np.concatenate(parts, 1)
    if not nempty:
      full = np.zeros((int(self.nnum[d]), out.shape[1]), np.float32)
      full[self.nempty_index(d)] = out
      out = full
    return out

  # octree.py:464-488 ------------------------------------------------------
  def search_key(self, query, depth, nempty=False):
    key = self.keys[depth]
    if nempty:
      key = key[self.nempty_index(depth)]
    idx = np.searchsorted(key, query).astype(I64)
    ok = idx < key.shape[0]
    found = np.zeros_like(ok)
    found[ok] = key[idx[ok]] == query[ok]
    idx[~found] = -1
    return idx


def normalize_points(points, bbmin, bbmax, scale):
  """ocnn/octree/points.py:223-244 applied to an fp32 array.  Python scalars
  act as fp32 when they meet an fp32 tensor, which numpy reproduces."""
  points = np.asarray(points, np.float32)
  box = bbmax - bbmin
  if isinstance(box, np.ndarray):
    box = float(box.max())
    bbmin = np.asarray(bbmin, np.float32)
  assert box > 0
  return ((points - bbmin) * (scale / box)).astype(np.float32)


def grow_full(oct, d):
  """octree.py:289-314."""
  num = 1 << (3 * d)
  B = oct.batch_size
  oct.nnum[d] = oct.nnum_nempty[d] = num * B
  key = np.arange(num, dtype=I64)[None, :] | (np.arange(B, dtype=I64)[:, None] << 48)
  oct.keys[d] = key.reshape(-1)
  oct.children[d] = np.arange(num * B, dtype=np.int32)


def build_octree(points, normals=None, features=None, batch_id=None,
                 depth=6, full_depth=2, batch_size=1, bbmin=-1.0, bbmax=1.0):
  """octree.py:201-287.  Returns (OctreeRef, idx) where idx maps each input
  point to its leaf (the inverse map of the unique)."""
  oct = OctreeRef(depth, full_depth, batch_size)
  pts = normalize_points(points, bbmin, bbmax, 2 ** depth)
  b = None if batch_size == 1 else np.asarray(batch_id).reshape(-1)
  key = xyz2key(pts[:, 0], pts[:, 1], pts[:, 2], b, depth)
  node_key, idx, counts = np.unique(key, return_inverse=True, return_counts=True)
  idx = idx.reshape(-1)

  for d in range(full_depth + 1):
    grow_full(oct, d)

  for d in range(depth, full_depth, -1):
    pkey_all = node_key >> 3
    head = np.ones(pkey_all.shape[0], bool)
    head[1:] = pkey_all[1:] != pkey_all[:-1]          # unique_consecutive
    pkey = pkey_all[head]
    pidx = np.cumsum(head) - 1
    oct.keys[d] = ((pkey[:, None] << 3) + np.arange(8, dtype=I64)).reshape(-1)
    oct.nnum[d] = oct.keys[d].shape[0]
    oct.nnum_nempty[d] = node_key.shape[0]
    children = -np.ones(oct.nnum[d], np.int32)
    children[(pidx << 3) | (node_key % 8)] = np.arange(node_key.shape[0], dtype=np.int32)
    oct.children[d] = children
    node_key = pkey if batch_size == 1 else \
        (((pkey >> 45) << 48) | (pkey & ((1 << 45) - 1)))

  d = full_depth
  children = -np.ones_like(oct.children[d])
  at = node_key if batch_size == 1 else \
      (((node_key >> 48) << (3 * d)) | (node_key & ((1 << 48) - 1)))
  children[at] = np.arange(node_key.shape[0], dtype=np.int32)
  oct.children[d] = children
  oct.nnum_nempty[d] = node_key.shape[0]

  # leaf signals: sequential fp32 scatter-add in point order, then mean
  nleaf = counts.shape[0]
  cnt = counts.astype(np.float32)[:, None]

  def seg_sum(v):
    out = np.zeros((nleaf, v.shape[1]), np.float32)
    np.add.at(out, idx, np.asarray(v, np.float32))
    return out

  oct.points[depth] = seg_sum(pts) / cnt
  if normals is not None:
    s = seg_sum(normals)
    nrm = np.sqrt((s * s).sum(1, keepdims=True, dtype=np.float32))
    oct.normals[depth] = s / np.maximum(nrm, np.float32(1e-12))
  if features is not None:
    oct.features[depth] = seg_sum(features) / cnt
  return oct, idx.astype(I64)


def construct_neigh(oct, d, force_lut=False):
  """octree.py:404-439."""
  if d <= oct.full_depth and not force_lut:
    nnum = 1 << (3 * d)
    key = np.arange(nnum, dtype=I64)
    x, y, z, _ = key2xyz(key, d)
    xyz = np.stack([x, y, z], -1)[:, None, :] + range_grid(-1, 1)[None]
    xyz = xyz.reshape(-1, 3)
    neigh = xyz2key(xyz[:, 0], xyz[:, 1], xyz[:, 2], depth=d)
    neigh = neigh[None, :] + np.arange(oct.batch_size, dtype=I64)[:, None] * nnum
    bound = 1 << d
    invalid = (xyz < 0).any(1) | (xyz >= bound).any(1)
    neigh[:, invalid] = -1
    oct.neighs[d] = neigh.reshape(-1, 27)
  else:
    lut_parent, lut_child = neigh_luts()
    child_p = oct.children[d - 1]
    neigh_p = oct.neighs[d - 1][child_p >= 0]       # (N, 27)
    neigh_p = neigh_p[:, lut_parent]                # (N, 8, 27)
    cp = child_p[neigh_p].astype(I64)               # -1 wraps to the last node
    invalid = (cp < 0) | (neigh_p < 0)
    neigh = cp * 8 + lut_child
    neigh[invalid] = -1
    oct.neighs[d] = neigh.reshape(-1, 27)


def construct_all_neigh(oct):
  for d in range(1, oct.depth + 1):                 # octree.py:441-446
    construct_neigh(oct, d)


def transpose_table(neigh, rows_in):
  """For a table T (R, K) with T[i,k] = j or -1, where every (j, k) pair has
  at most one i, returns Tt (rows_in, K) with Tt[j, k] = i.  This turns the
  scatter ``gin[T[i,k]] += f(i,k)`` (octree_conv.py:160-166) into a gather."""
  R, K = neigh.shape
  out = -np.ones((rows_in, K), I64)
  i, k = np.nonzero(neigh >= 0)
  j = neigh[i, k]
  assert np.all(out[j, k] == -1)
  out[j, k] = i
  return out
