"""Pins the numpy oracle of the octree build / neighbour search against the
data files held by the reference's own tests (copied as data under
tests/golden/ref_data) and against closed forms.  CPU only."""

import os

import numpy as np
import pytest

from oracle import octree_ref as R


def load(ref_data, name):
  return np.load(os.path.join(ref_data, name))


def single_octree(ref_data, i):
  d = load(ref_data, 'octree/test_%03d.npz' % i)
  oct, idx = R.build_octree(d['points'], d['normals'], depth=int(d['depth']),
                            full_depth=int(d['full_depth']))
  return oct, idx, d


def batch_octree(ref_data):
  d4 = load(ref_data, 'octree/test_004.npz')
  d5 = load(ref_data, 'octree/test_005.npz')
  pts = np.concatenate([d4['points'], d5['points']])
  nrm = np.concatenate([d4['normals'], d5['normals']])
  bid = np.concatenate([np.zeros(len(d4['points']), np.float32),
                        np.ones(len(d5['points']), np.float32)])
  d = load(ref_data, 'batch_45.npz')
  oct, idx = R.build_octree(pts, nrm, batch_id=bid, depth=int(d['depth']),
                            full_depth=int(d['full_depth']), batch_size=2)
  return oct, d


# ---- Morton keys ----------------------------------------------------------

def interleave_closed_form(x, y, z, depth):
  key = 0
  for i in range(depth):
    key |= ((x >> i) & 1) << (3 * i + 2)
    key |= ((y >> i) & 1) << (3 * i + 1)
    key |= ((z >> i) & 1) << (3 * i)
  return key


@pytest.mark.parametrize('depth', [1, 3, 5, 8, 9, 12, 16])
def test_xyz2key_closed_form(depth):
  rng = np.random.default_rng(depth)
  n = 200
  xyz = rng.integers(0, 1 << depth, size=(n, 3))
  b = rng.integers(0, 32768, size=n)
  key = R.xyz2key(xyz[:, 0], xyz[:, 1], xyz[:, 2], b, depth)
  for i in range(n):
    want = interleave_closed_form(int(xyz[i, 0]), int(xyz[i, 1]), int(xyz[i, 2]), depth)
    assert int(key[i]) == (int(b[i]) << 48) | want


def test_key_axis_convention():
  # x is the most significant bit of each 3-bit group, z the least.
  assert R.xyz2key(np.array([1]), np.array([0]), np.array([0]), depth=4)[0] == 4
  assert R.xyz2key(np.array([0]), np.array([1]), np.array([0]), depth=4)[0] == 2
  assert R.xyz2key(np.array([0]), np.array([0]), np.array([1]), depth=4)[0] == 1


def test_key_roundtrip_like_reference_test():
  # the reference's round-trip property: 16-bit coordinates, 15-bit batch
  rng = np.random.default_rng(0)
  xyz = rng.integers(0, 2 ** 16, size=(1000, 3))
  b = rng.integers(0, 2 ** 15, size=1000)
  key = R.xyz2key(xyz[:, 0], xyz[:, 1], xyz[:, 2], b, 16)
  x, y, z, bb = R.key2xyz(key, 16)
  assert np.array_equal(x, xyz[:, 0]) and np.array_equal(y, xyz[:, 1])
  assert np.array_equal(z, xyz[:, 2]) and np.array_equal(bb, b)


def test_key_out_of_range_wraps():
  # negative and too-large coordinates are masked, not rejected
  k = R.xyz2key(np.array([-1.0, 32.0, -0.5]), np.array([0.0, 0.0, 0.0]),
                np.array([0.0, 0.0, 0.0]), depth=5)
  assert k[0] == interleave_closed_form(31, 0, 0, 5)
  assert k[1] == 0 and k[2] == 0


# ---- build ----------------------------------------------------------------

def test_three_point_known_answer():
  # literal values of the reference's 3-point test (test/test_octree.py:19-85)
  pts = np.array([[-1, -1, -1], [0, 0, -1], [0.0625, 0.0625, -1]], np.float32)
  nrm = np.array([[1, 0, 0], [-1, 0, 0], [0, 1, 0]], np.float32)
  fea = np.array([[1, -1], [2, -2], [3, -3]], np.float32)
  oct, idx = R.build_octree(pts, nrm, fea, depth=5, full_depth=1)
  assert oct.nnum.tolist() == [1, 8, 16, 16, 16, 16]
  assert oct.nnum_nempty.tolist() == [1, 2, 2, 2, 2, 3]
  tails = [None, None, 48, 384, 3072, 24576]
  for d in range(2, 6):
    want = list(range(8)) + list(range(tails[d], tails[d] + 8))
    assert oct.keys[d].tolist() == want
  assert oct.children[1].tolist() == [0, -1, -1, -1, -1, -1, 1, -1]
  for d in (2, 3, 4):
    assert oct.children[d].tolist() == [0] + [-1] * 7 + [1] + [-1] * 7
  assert oct.children[5].tolist() == [0] + [-1] * 7 + [1] + [-1] * 5 + [2, -1]
  assert [oct.nempty_index(d).tolist() for d in range(6)] == \
      [[0], [0, 6], [0, 8], [0, 8], [0, 8], [0, 8, 14]]
  assert np.array_equal(oct.normals[5], nrm)
  assert np.array_equal(oct.features[5], fea)
  assert idx.tolist() == [0, 1, 2]


@pytest.mark.parametrize('i', [1, 2, 3, 4, 5])
def test_build_against_reference_fixture(ref_data, i):
  oct, idx, d = single_octree(ref_data, i)
  assert np.array_equal(oct.nnum, d['nnum'])
  assert np.array_equal(oct.nnum_nempty, d['nnum_nempty'])
  assert np.array_equal(np.concatenate(oct.keys), d['key'])
  assert np.array_equal(np.concatenate(oct.children), d['child'])
  assert oct.children[0].dtype == np.int32 and oct.keys[0].dtype == np.int64
  assert np.allclose(oct.normals[oct.depth], d['feature'][:, :3])
  # invariants
  for dd in range(oct.full_depth + 1, oct.depth + 1):
    assert np.all(np.diff(oct.keys[dd]) > 0)
    assert oct.nnum[dd] == 8 * oct.nnum_nempty[dd - 1]
    c = oct.children[dd]
    assert np.array_equal(c[c >= 0], np.arange(oct.nnum_nempty[dd]))


def test_batched_build_against_reference_fixture(ref_data):
  oct, d = batch_octree(ref_data)
  assert np.array_equal(oct.nnum, d['nnum'])
  assert np.array_equal(oct.nnum_nempty, d['nnum_nempty'])
  assert np.array_equal(np.concatenate(oct.keys), d['key'])
  assert np.array_equal(np.concatenate(oct.children), d['child'])
  assert np.allclose(oct.normals[oct.depth], d['feature'][:, :3])


# ---- neighbours -----------------------------------------------------------

def test_neigh_against_reference_fixture(ref_data):
  oct, d = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  got = np.concatenate(oct.neighs[1:], 0)
  assert got.dtype == np.int64
  assert np.array_equal(got, d['neigh'])


def test_neigh_branches_agree(ref_data):
  # the reference's own invariant (test/test_octree.py:181-191)
  oct, _ = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  full = oct.neighs[3].copy()
  R.construct_neigh(oct, 3, force_lut=True)
  assert np.array_equal(full, oct.neighs[3])


def brute_force_neigh(oct, d):
  key = oct.keys[d]
  x, y, z, b = R.key2xyz(key, d)
  out = -np.ones((len(key), 27), np.int64)
  grid = R.range_grid(-1, 1)
  for k in range(27):
    xx, yy, zz = x + grid[k, 0], y + grid[k, 1], z + grid[k, 2]
    ok = (xx >= 0) & (yy >= 0) & (zz >= 0) & (xx < (1 << d)) & (yy < (1 << d)) & (zz < (1 << d))
    q = R.xyz2key(xx, yy, zz, b, d)
    pos = np.searchsorted(key, q)
    pos[pos >= len(key)] = 0
    hit = ok & (key[pos] == q)
    out[hit, k] = pos[hit]
  return out


@pytest.mark.parametrize('d', [2, 4, 6])
def test_neigh_brute_force(ref_data, d):
  oct, _ = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  assert np.array_equal(oct.neighs[d], brute_force_neigh(oct, d))


def test_neigh_invariants(ref_data):
  oct, _ = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  for d in range(1, oct.depth + 1):
    n = oct.neighs[d]
    assert np.array_equal(n[:, 13], np.arange(n.shape[0]))
    i, k = np.nonzero(n >= 0)
    assert np.array_equal(n[n[i, k], 26 - k], i)      # central symmetry
    assert n.max() < oct.nnum[d]


def test_get_neigh_closed_forms(ref_data):
  oct, _ = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  for d in range(1, oct.depth + 1):
    t = oct.get_neigh(d, '222', 2, False)
    assert np.array_equal(t, (np.arange(t.shape[0]) * 8)[:, None] + np.arange(8))
  d = 5
  # non-empty tables: brute force on the non-empty keys
  ne = oct.nempty_index(d)
  key = oct.keys[d][ne]
  t = oct.get_neigh(d, '333', 1, True)
  bf = brute_force_neigh(oct, d)[ne]
  want = -np.ones_like(bf)
  v = bf >= 0
  rank = -np.ones(oct.nnum[d], np.int64)
  rank[ne] = np.arange(len(ne))
  want[v] = rank[bf[v]]
  assert np.array_equal(t, want)
  assert t.shape[0] == len(key)
  # column selection
  for kern, cols in R.LUT_KERNEL.items():
    assert np.array_equal(oct.get_neigh(d, kern, 1, False), oct.neighs[d][:, cols])
  with pytest.raises(ValueError):
    oct.get_neigh(d, '123')
  with pytest.raises(ValueError):
    oct.get_neigh(d, '333', 3)


def test_transpose_table(ref_data):
  oct, _ = batch_octree(ref_data)
  R.construct_all_neigh(oct)
  d = 5
  # stride 1: the transposed table is the mirrored table
  t = oct.get_neigh(d, '333', 1, False)
  assert np.array_equal(R.transpose_table(t, oct.nnum[d]), t[:, ::-1])
  # stride 2, 3x3x3: every (input row, slot) has at most one producer
  t = oct.get_neigh(d, '333', 2, True)
  tt = R.transpose_table(t, int(oct.nnum_nempty[d]))
  i, k = np.nonzero(t >= 0)
  assert np.array_equal(tt[t[i, k], k], i)
  assert (tt >= 0).sum() == (t >= 0).sum()


def test_search_key_fixture(ref_data):
  oct, _ = batch_octree(ref_data)
  d = load(ref_data, 'search_key.npz')
  q = d['xyzb'].astype(np.int64)
  key = R.xyz2key(q[:, 0], q[:, 1], q[:, 2], q[:, 3], 5)
  assert np.array_equal(oct.search_key(key, 5, False), d['idx'])
  assert np.array_equal(oct.search_key(key, 5, True), d['idx_ne'])


@pytest.mark.parametrize('i', [1, 2, 3, 4, 5])
def test_input_feature_against_reference_fixture(ref_data, i):
  """get_input_feature('ND') (ocnn/octree/octree.py:525-568) on the reference's octree files:
  their `feature` array holds the leaf normals and, in its fourth column, the displacement
  <local point, normal> as the tool that wrote the files scaled it, by 2 / sqrt(3) (the current
  Python code of the reference has no such factor).  Pins the leaf averages of the points, the
  local coordinates and the order of the channels."""
  d = np.load(os.path.join(ref_data, 'octree/test_%03d.npz' % i))
  w, _ = R.build_octree(d['points'], d['normals'], None, None, int(d['depth']), int(d['full_depth']), 1)
  f = w.get_input_feature('ND', nempty=True)
  assert f.shape == d['feature'].shape and f.dtype == np.float32
  assert np.allclose(f[:, :3], d['feature'][:, :3])
  assert np.abs(d['feature'][:, 3] - 2.0 / np.sqrt(3.0) * f[:, 3]).max() < 2e-6
  full = w.get_input_feature('ND', nempty=False)
  assert full.shape[0] == int(d['nnum'][-1]) and np.array_equal(full[w.nempty_index(w.depth)], f)
  assert not full[w.children[w.depth] < 0].any()
