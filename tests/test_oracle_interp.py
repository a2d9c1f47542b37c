"""Pins the numpy oracle of point interpolation, upsampling and max pooling against the data
file held by the reference's own interpolation test (interp.npz, copied as data under
tests/golden/ref_data) and against what the mathematics fixes.  CPU only."""

import numpy as np
import pytest
import torch

from oracle import interp_ref as I
from oracle import octree_ref as R
from test_oracle_octree import batch_octree, load


def test_interp_against_reference_fixture(ref_data):
  """test/test_octree_interp.py:21-43: the same four calls, the same tolerance."""
  oct, _ = batch_octree(ref_data)
  t = load(ref_data, 'interp.npz')
  depth = 5
  data, pts = t['data'], t['pts']
  data_ne = I.octree_depad(oct, data, depth)
  assert np.allclose(I.linear_pts(oct, data, depth, pts, False), t['linear'], atol=1e-6)
  assert np.allclose(I.linear_pts(oct, data_ne, depth, pts, True), t['linear_ne'], atol=1e-6)
  assert np.allclose(I.nearest_pts(oct, data, depth, pts, False), t['near'], atol=1e-6)
  assert np.allclose(I.nearest_pts(oct, data_ne, depth, pts, True), t['near_ne'], atol=1e-6)


@pytest.mark.parametrize('nempty', [False, True])
def test_nearest_upsample_is_nearest_pts_at_child_centres(ref_data, nempty):
  """test/test_octree_interp.py:45-73."""
  oct, _ = batch_octree(ref_data)
  depth = 4
  rows = int(oct.nnum_nempty[depth] if nempty else oct.nnum[depth])
  data = np.random.default_rng(0).random((rows, 4), dtype=np.float32)
  out = I.nearest_upsample(oct, data, depth, nempty)
  x, y, z, b = I.xyzb(oct, depth + 1, nempty)
  pts = np.stack([x, y, z, b], 1).astype(np.float32)
  pts[:, :3] = (pts[:, :3] + 0.5) * 0.5
  assert np.array_equal(out, I.nearest_pts(oct, data, depth, pts, nempty, bound_check=True))
  assert np.array_equal(out, I.upsample(oct, data, depth, depth + 1, 'nearest', nempty))


def test_linear_weights_on_a_full_layer(ref_data):
  """On a full layer every neighbour inside the volume exists: the weights of an interior
  point sum to one, a linear field is reproduced exactly (to rounding), and a point at a
  voxel centre takes that voxel's value."""
  oct, _ = batch_octree(ref_data)
  depth = 3                                       # full layer of the fixture octree
  assert oct.nnum[depth] == 2 * 8 ** depth
  rng = np.random.default_rng(1)
  n = 500
  pts = np.concatenate([rng.uniform(0.6, 2 ** depth - 0.6, (n, 3)), rng.integers(0, 2, (n, 1))], 1).astype(np.float32)
  idx, w = I.linear_weights(oct, depth, pts)
  assert (idx >= 0).all() and np.allclose(w.sum(1), 1.0, atol=1e-6)
  x, y, z, b = I.xyzb(oct, depth)
  field = (0.3 * x - 0.7 * y + 0.2 * z + 5.0 * b + 1.0).astype(np.float32)[:, None]
  want = 0.3 * (pts[:, 0] - 0.5) - 0.7 * (pts[:, 1] - 0.5) + 0.2 * (pts[:, 2] - 0.5) + 5.0 * pts[:, 3] + 1.0
  assert np.allclose(I.linear_pts(oct, field, depth, pts)[:, 0], want, atol=1e-5)
  centres = np.stack([x + 0.5, y + 0.5, z + 0.5, b], 1).astype(np.float32)
  data = rng.random((int(oct.nnum[depth]), 3), dtype=np.float32)
  assert np.allclose(I.linear_pts(oct, data, depth, centres), data, atol=1e-6)
  assert np.array_equal(I.nearest_pts(oct, data, depth, centres), data)


def test_linear_is_normalised_where_neighbours_are_missing(ref_data):
  """Sparse level: a constant field interpolates to that constant wherever at least one
  neighbour exists, and to zero where none does; bound_check drops what lies outside."""
  oct, _ = batch_octree(ref_data)
  depth = 5
  t = load(ref_data, 'interp.npz')
  pts = t['pts']
  idx, w = I.linear_weights(oct, depth, pts, nempty=True)
  ones = np.full((int(oct.nnum_nempty[depth]), 1), 3.0, np.float32)
  out = I.linear_pts(oct, ones, depth, pts, nempty=True)[:, 0]
  some = (idx >= 0).any(1)
  assert some.any() and np.allclose(out[some], 3.0, atol=1e-5) and np.all(out[~some] == 0)
  far = pts.copy()
  far[:, 0] += 2 ** depth                          # outside the volume: keys wrap, bounds do not
  assert np.all(I.linear_pts(oct, ones, depth, far, True, bound_check=True) == 0)
  assert np.all(I.nearest_pts(oct, ones, depth, far, True, bound_check=True) == 0)


def test_linear_grad_is_the_adjoint(ref_data):
  oct, _ = batch_octree(ref_data)
  depth = 5
  t = load(ref_data, 'interp.npz')
  pts = t['pts'][:2000]
  rng = np.random.default_rng(2)
  rows = int(oct.nnum[depth])
  data = rng.standard_normal((rows, 3)).astype(np.float32)
  grad = rng.standard_normal((len(pts), 3)).astype(np.float32)
  lhs = (I.linear_pts(oct, data, depth, pts).astype(np.float64) * grad).sum()
  rhs = (I.linear_pts_grad(oct, grad, depth, pts, rows) * data).sum()
  assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))


def test_upsample_linear_two_levels(ref_data):
  """OctreeUpsample over two levels = linear_pts at the centres of the target nodes."""
  oct, _ = batch_octree(ref_data)
  depth, target = 3, 5
  data = np.random.default_rng(3).random((int(oct.nnum[depth]), 2), dtype=np.float32)
  out = I.upsample(oct, data, depth, target, 'linear', False)
  assert out.shape == (int(oct.nnum[target]), 2)
  x, y, z, b = I.xyzb(oct, target)
  pts = np.stack([(x + 0.5) / 4, (y + 0.5) / 4, (z + 0.5) / 4, b], 1).astype(np.float32)
  assert np.array_equal(out, I.linear_pts(oct, data, depth, pts))


def test_max_pool_on_a_full_layer_is_max_pool3d(ref_data):
  """Full layer: the 8 children of a node are a 2x2x2 block of the voxel grid, so the pooled
  values are torch.nn.functional.max_pool3d of the grid."""
  oct, _ = batch_octree(ref_data)
  depth = 3
  n = 2 ** depth
  rng = np.random.default_rng(4)
  data = rng.standard_normal((int(oct.nnum[depth]), 5)).astype(np.float32)
  out, idx = I.max_pool(oct, data, depth, nempty=False)
  x, y, z, b = I.xyzb(oct, depth)
  grid = np.zeros((2, 5, n, n, n), np.float32)
  grid[b, :, x, y, z] = data
  pooled = torch.nn.functional.max_pool3d(torch.from_numpy(grid), 2).numpy()
  xp, yp, zp, bp = I.xyzb(oct, depth - 1)
  assert np.array_equal(out, pooled[bp, :, xp, yp, zp])
  # unpooling puts each maximum back where it came from
  up = I.max_unpool(oct, out, idx, depth - 1, nempty=False)
  assert np.array_equal((up != 0).sum(), (out != 0).sum())
  assert np.array_equal(np.take_along_axis(up.reshape(-1, 8, 5), idx[:, None, :], 1)[:, 0], out)


@pytest.mark.parametrize('nempty', [False, True])
def test_max_pool_on_a_sparse_level(ref_data, nempty):
  """Sparse level against a loop over parents and children."""
  oct, _ = batch_octree(ref_data)
  depth = 5
  rows = int(oct.nnum_nempty[depth] if nempty else oct.nnum[depth])
  data = np.random.default_rng(5).standard_normal((rows, 3)).astype(np.float32)
  out, idx = I.max_pool(oct, data, depth, nempty)
  child = oct.children[depth]
  parents = oct.nempty_index(depth - 1)
  assert idx.shape == (len(parents), 3)
  for p in range(0, len(parents), 37):
    rows8 = []
    for j in range(8):
      q = 8 * p + j
      if nempty:
        rows8.append(data[child[q]] if child[q] >= 0 else np.full(3, -np.inf, np.float32))
      else:
        rows8.append(data[q])
    want = np.max(np.stack(rows8), 0)
    got = out[p] if nempty else out[parents[p]]
    assert np.array_equal(got, want)
  if not nempty:
    empty = np.setdiff1d(np.arange(int(oct.nnum[depth - 1])), parents)
    assert np.all(out[empty] == 0)
  up = I.max_unpool(oct, out, idx, depth - 1, nempty)
  assert up.shape == data.shape
  hit = up != 0
  assert np.array_equal(up[hit], data[hit])
