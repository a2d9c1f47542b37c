"""Numpy restatement of the reference's point interpolation, nearest upsampling and
2x2x2 max pooling on octrees.

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this file.

Every function names the reference lines it follows (paths relative to the reference
checkout).  Floating-point work is done in fp32 with the reference's operation order where
that order is visible in its source; the sum over the (at most 8) neighbours of a point runs
in the order of the neighbour grid, where the reference leaves it to torch.sparse.mm.

Pinned by: interp.npz of the reference's tests (nearest and linear, all nodes and non-empty
nodes), the reference's own identity nearest_upsample == nearest_pts at the child centres,
partition of unity and exactness on linear fields for the linear weights,
torch.nn.functional.max_pool3d on full layers for the pooling.
"""

import numpy as np

from . import octree_ref as R

F32 = np.float32
GRID = np.array([[0, 0, 0], [0, 0, 1], [0, 1, 0], [0, 1, 1],
                 [1, 0, 0], [1, 0, 1], [1, 1, 0], [1, 1, 1]], dtype=np.int64)


def search_xyzb(oct, query, depth, nempty=False):
  """ocnn/octree/octree.py:448-462: Morton key of (x, y, z, b) (truncated to integers,
  masked like any key), then the binary search of search_key."""
  key = R.xyz2key(query[:, 0], query[:, 1], query[:, 2], query[:, 3], depth)
  return oct.search_key(key, depth, nempty)


def xyzb(oct, depth, nempty=False):
  """ocnn/octree/octree.py:122-137."""
  key = oct.keys[depth]
  if nempty:
    key = key[oct.nempty_index(depth)]
  return R.key2xyz(key, depth)


def octree_depad(oct, data, depth):
  return data[oct.nempty_index(depth)]


def octree_pad(oct, data, depth, val=0.0):
  out = np.full((int(oct.nnum[depth]), data.shape[1]), val, data.dtype)
  out[oct.nempty_index(depth)] = data
  return out


def nearest_pts(oct, data, depth, pts, nempty=False, bound_check=False):
  """ocnn/nn/octree_interp.py:15-46."""
  idx = search_xyzb(oct, pts, depth, nempty)
  valid = idx > -1
  if bound_check:
    valid &= ((pts[:, :3] >= 0) & (pts[:, :3] < 2 ** depth)).all(1)
  out = np.zeros((pts.shape[0], data.shape[1]), data.dtype)
  out[valid] = data[idx[valid]]
  return out


def linear_weights(oct, depth, pts, nempty=False, bound_check=False):
  """ocnn/nn/octree_interp.py:60-88: the 8 neighbour rows (-1 = none) and fp32 weights of every
  point.  Values sit at voxel centres: xyzf = p - 0.5, integer part by floor, weights
  |prod_d((1 - g_d) - frac_d)|."""
  pts = pts.astype(F32)
  xyzf = pts[:, :3] - F32(0.5)
  xyzi = np.floor(xyzf)
  frac = xyzf - xyzi
  n = pts.shape[0]
  xyzn = (xyzi[:, None, :] + GRID[None].astype(F32)).reshape(-1, 3)
  batch = np.repeat(pts[:, 3:4], 8, axis=1).reshape(-1, 1)
  idx = search_xyzb(oct, np.concatenate([xyzn, batch], 1), depth, nempty)
  valid = idx > -1
  if bound_check:
    valid &= ((xyzn >= 0) & (xyzn < 2 ** depth)).all(1)
  t = (F32(1.0) - GRID[None].astype(F32)) - frac[:, None, :]          # (N, 8, 3)
  w = np.abs((t[:, :, 0] * t[:, :, 1]) * t[:, :, 2]).astype(F32)      # prod over the last axis
  idx = np.where(valid, idx, -1).reshape(n, 8)
  w = np.where(valid.reshape(n, 8), w, F32(0))
  return idx, w


def linear_pts(oct, data, depth, pts, nempty=False, bound_check=False):
  """ocnn/nn/octree_interp.py:49-103: out = (sum_j w_j data[idx_j]) / (sum_j w_j + 1e-12)."""
  idx, w = linear_weights(oct, depth, pts, nempty, bound_check)
  out = np.zeros((pts.shape[0], data.shape[1]), F32)
  norm = np.zeros((pts.shape[0], 1), F32)
  for j in range(8):
    v = idx[:, j] >= 0
    out[v] += w[v, j:j + 1] * data[idx[v, j]].astype(F32)
    norm[v, 0] += w[v, j]
  return (out / (norm + F32(1e-12))).astype(data.dtype)


def linear_pts_grad(oct, grad, depth, pts, rows, nempty=False, bound_check=False):
  """Gradient of linear_pts with respect to data (autograd of the two sparse products and
  the division): gdata[idx_j] += w_j * grad / (norm + 1e-12)."""
  idx, w = linear_weights(oct, depth, pts, nempty, bound_check)
  norm = w.sum(1, dtype=np.float64)[:, None]
  gs = grad.astype(np.float64) / (norm + 1e-12)
  out = np.zeros((rows, grad.shape[1]), np.float64)
  for j in range(8):
    v = idx[:, j] >= 0
    np.add.at(out, idx[v, j], w[v, j:j + 1].astype(np.float64) * gs[v])
  return out


def nearest_upsample(oct, data, depth, nempty=False):
  """ocnn/nn/octree_interp.py:135-158: every child takes its parent's row."""
  out = data
  if not nempty:
    out = octree_depad(oct, out, depth)
  out = np.repeat(out[:, None, :], 8, axis=1).reshape(-1, data.shape[1])
  if nempty:
    out = octree_depad(oct, out, depth + 1)
  return out


def upsample(oct, data, depth, target_depth=None, method='linear', nempty=False):
  """ocnn/nn/octree_interp.py:161-193 (OctreeUpsample.forward)."""
  if target_depth is None:
    target_depth = depth + 1
  if target_depth == depth:
    return data
  if target_depth == depth + 1 and method == 'nearest':
    return nearest_upsample(oct, data, depth, nempty)
  x, y, z, b = xyzb(oct, target_depth, nempty)
  pts = np.stack([x, y, z, b], 1).astype(F32)
  pts[:, :3] = (pts[:, :3] + F32(0.5)) * F32(2.0 ** (depth - target_depth))
  fn = linear_pts if method == 'linear' else nearest_pts
  return fn(oct, data, depth, pts, nempty)


def max_pool(oct, data, depth, nempty=False):
  """ocnn/nn/octree_pool.py:16-37: maximum over the 8 children (first one on ties) and its
  index; empty children count as -inf (non-empty form) / the output is zero-padded to all
  nodes of depth - 1 (all-nodes form)."""
  if nempty:
    data = octree_pad(oct, data, depth, -np.inf)
  d3 = data.reshape(-1, 8, data.shape[1])
  idx = d3.argmax(1).astype(np.int64)
  out = np.take_along_axis(d3, idx[:, None, :], 1)[:, 0, :]
  if not nempty:
    out = octree_pad(oct, out, depth - 1)
  return out, idx


def max_unpool(oct, data, idx, depth, nempty=False):
  """ocnn/nn/octree_pool.py:40-65: data of depth -> depth + 1, each value to the child that
  gave the maximum, zeros elsewhere."""
  if not nempty:
    data = octree_depad(oct, data, depth)
  n, c = data.shape
  out = np.zeros((n, 8, c), data.dtype)
  np.put_along_axis(out, idx[:, None, :], data[:, None, :], 1)
  out = out.reshape(-1, c)
  if nempty:
    out = octree_depad(oct, out, depth + 1)
  return out
