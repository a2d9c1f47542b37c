"""GPU parity of the octree build and neighbour search: the HIP path (through the
C ABI) against the reference's data files and the numpy oracle, bit exact."""

import os
import sys

import numpy as np
import pytest
from conftest import random_cases
import torch

import ocnn_amd
from ocnn_amd import synthetic
from ocnn_amd.octree import Octree, Points, key2xyz, merge_octrees, merge_points, xyz2key
from oracle import octree_ref as R

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def np_(t):
  return t.detach().cpu().numpy()


def fixture_points(ref_data, i):
  d = np.load(os.path.join(ref_data, 'octree/test_%03d.npz' % i))
  pc = Points(torch.from_numpy(d['points']).to(DEV), torch.from_numpy(d['normals']).to(DEV))
  return pc, d


def fixture_octree(ref_data, i):
  pc, d = fixture_points(ref_data, i)
  o = Octree(int(d['depth']), int(d['full_depth']))
  idx = o.build_octree(pc)
  return o, idx, d


def check_against(o, d):
  assert np.array_equal(o.nnum.numpy(), d['nnum'])
  assert np.array_equal(o.nnum_nempty.numpy(), d['nnum_nempty'])
  key = np_(torch.cat(o.keys))
  child = np_(torch.cat(o.children))
  assert key.dtype == np.int64 and child.dtype == np.int32
  assert np.array_equal(key, d['key'])
  assert np.array_equal(child, d['child'])
  assert np.allclose(np_(o.normals[o.depth]), d['feature'][:, :3])


def test_keys_gpu_vs_oracle():
  say('keys: random 16-bit coordinates')
  g = torch.Generator().manual_seed(0)
  for depth in (3, 8, 9, 16):
    xyz = torch.randint(-2, (1 << depth) + 2, (5000, 3), generator=g)
    b = torch.randint(0, 32768, (5000,), generator=g)
    key = xyz2key(xyz[:, 0].to(DEV), xyz[:, 1].to(DEV), xyz[:, 2].to(DEV), b.to(DEV), depth)
    want = R.xyz2key(xyz[:, 0].numpy(), xyz[:, 1].numpy(), xyz[:, 2].numpy(), b.numpy(), depth)
    assert np.array_equal(np_(key), want)
    x, y, z, bb = key2xyz(key, depth)
    wx, wy, wz, wb = R.key2xyz(want, depth)
    assert np.array_equal(np_(x), wx) and np.array_equal(np_(y), wy)
    assert np.array_equal(np_(z), wz) and np.array_equal(np_(bb), wb)
  # float inputs truncate toward zero; scalar batch; no batch
  f = torch.tensor([0.9, 1.1, -0.5, 3.99], device=DEV)
  assert np.array_equal(np_(xyz2key(f, f, f, 3, 4)),
                        R.xyz2key(np_(f), np_(f), np_(f), np.full(4, 3), 4))
  assert np.array_equal(np_(xyz2key(f, f, f, depth=4)), R.xyz2key(np_(f), np_(f), np_(f), None, 4))
  # empty input
  e = torch.zeros(0, device=DEV)
  assert xyz2key(e, e, e, depth=4).numel() == 0


def test_three_point_known_answer():
  say('build: 3-point literal case')
  pts = torch.tensor([[-1, -1, -1], [0, 0, -1], [0.0625, 0.0625, -1]], dtype=torch.float32)
  nrm = torch.tensor([[1, 0, 0], [-1, 0, 0], [0, 1, 0]], dtype=torch.float32)
  fea = torch.tensor([[1, -1], [2, -2], [3, -3]], dtype=torch.float32)
  o = Octree(depth=5, full_depth=1, device=DEV)
  idx = o.build_octree(Points(pts.to(DEV), nrm.to(DEV), fea.to(DEV)))
  assert o.nnum.tolist() == [1, 8, 16, 16, 16, 16]
  assert o.nnum_nempty.tolist() == [1, 2, 2, 2, 2, 3]
  tails = {2: 48, 3: 384, 4: 3072, 5: 24576}
  for d in range(2, 6):
    assert np_(o.keys[d]).tolist() == list(range(8)) + list(range(tails[d], tails[d] + 8))
  assert np_(o.children[1]).tolist() == [0, -1, -1, -1, -1, -1, 1, -1]
  assert np_(o.children[5]).tolist() == [0] + [-1] * 7 + [1] + [-1] * 5 + [2, -1]
  assert [np_(o.nempty_index(d)).tolist() for d in range(6)] == \
      [[0], [0, 6], [0, 8], [0, 8], [0, 8], [0, 8, 14]]
  assert torch.equal(o.normals[5].cpu(), nrm) and torch.equal(o.features[5].cpu(), fea)
  assert np_(idx).tolist() == [0, 1, 2]
  for d in range(6):
    assert torch.equal(o.nempty_mask(d), o.children[d] >= 0)


@pytest.mark.parametrize('i', [1, 2, 3, 4, 5])
def test_build_against_reference_fixture(ref_data, i):
  say('build: reference fixture', i)
  o, idx, d = fixture_octree(ref_data, i)
  check_against(o, d)
  want, widx = R.build_octree(d['points'], d['normals'], depth=int(d['depth']),
                              full_depth=int(d['full_depth']))
  assert np.array_equal(np_(idx), widx)
  assert np.array_equal(np_(o.points[o.depth]), want.points[o.depth])     # same sum order
  assert np.allclose(np_(o.normals[o.depth]), want.normals[o.depth], atol=1e-6)


def batched_points(ref_data):
  p4, _ = fixture_points(ref_data, 4)
  p5, _ = fixture_points(ref_data, 5)
  return merge_points([p4, p5])


def test_batched_build_against_reference_fixture(ref_data):
  say('build: batch of two, reference fixture')
  d = np.load(os.path.join(ref_data, 'batch_45.npz'))
  o = Octree(int(d['depth']), int(d['full_depth']), batch_size=2)
  o.build_octree(batched_points(ref_data))
  check_against(o, d)
  o.construct_all_neigh()
  neigh = torch.cat(o.neighs[1:], dim=0)
  assert neigh.dtype == torch.long
  assert np.array_equal(np_(neigh), d['neigh'])


def merged_octree(ref_data):
  o4, _, _ = fixture_octree(ref_data, 4)
  o5, _, _ = fixture_octree(ref_data, 5)
  o = merge_octrees([o4, o5])
  o.construct_all_neigh()
  return o


def test_merge_and_neigh_against_reference_fixture(ref_data):
  say('neigh: merged octrees, reference fixture')
  d = np.load(os.path.join(ref_data, 'batch_45.npz'))
  o = merged_octree(ref_data)
  check_against(o, d)
  assert np.array_equal(np_(torch.cat(o.neighs[1:], dim=0)), d['neigh'])
  assert o.batch_nnum.sum(1).tolist() == o.nnum.tolist()
  # moving to the host keeps every table
  c = o.to('cpu')
  assert np.array_equal(torch.cat(c.neighs[1:], dim=0).numpy(), d['neigh'])
  assert np.array_equal(torch.cat(c.keys).numpy(), d['key'])


def test_neigh_branches_agree(ref_data):
  say('neigh: full-layer branch == parent branch at depth 3')
  o = merged_octree(ref_data)
  full = o.neighs[3].clone()
  o.full_depth = 2
  o.construct_neigh(3)
  assert torch.equal(full, o.neighs[3])


def oracle_batch(ref_data):
  d4 = np.load(os.path.join(ref_data, 'octree/test_004.npz'))
  d5 = np.load(os.path.join(ref_data, 'octree/test_005.npz'))
  pts = np.concatenate([d4['points'], d5['points']])
  nrm = np.concatenate([d4['normals'], d5['normals']])
  bid = np.concatenate([np.zeros(len(d4['points'])), np.ones(len(d5['points']))])
  o, _ = R.build_octree(pts, nrm, batch_id=bid, depth=6, full_depth=3, batch_size=2)
  R.construct_all_neigh(o)
  return o


KERNELS = ['333', '222', '311', '131', '113', '331', '313', '133']


def test_get_neigh_grid_vs_oracle(ref_data):
  say('get_neigh: 8 kernels x 2 strides x nempty, depths 3..6')
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  for d in (3, 4, 5, 6):
    for kern in KERNELS:
      for stride in (1, 2):
        for ne in (False, True):
          got = o.get_neigh(d, kern, stride, ne)
          assert got.dtype == torch.long
          assert np.array_equal(np_(got), w.get_neigh(d, kern, stride, ne)), (d, kern, stride, ne)
          t32 = o._table(d, kern, stride, ne)
          assert t32.dtype == torch.int32 and np.array_equal(np_(t32), np_(got))
    assert np.array_equal(np_(o.nempty_index(d)), w.nempty_index(d))
    assert np.array_equal(np_(o.nempty_neigh(d)), w.nempty_neigh(d))
  assert o.get_neigh(5) is o.get_neigh(5)                 # the cached tensor itself
  assert o.get_neigh(5, '222', 2) is not o.get_neigh(5, '222', 2)
  with pytest.raises(ValueError):
    o.get_neigh(5, '223')
  with pytest.raises(ValueError):
    o.get_neigh(5, '333', 4)


def test_inverse_table_vs_oracle(ref_data):
  say('inverse tables')
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  d = 5
  for kern, stride, ne in [('333', 2, True), ('333', 2, False), ('222', 2, True),
                           ('222', 1, False), ('313', 2, True)]:
    rows_in = int(w.nnum_nempty[d] if ne else w.nnum[d])
    got = o._table_t(d, kern, stride, ne, rows_in)
    want = R.transpose_table(w.get_neigh(d, kern, stride, ne), rows_in)
    assert np.array_equal(np_(got), want), (kern, stride, ne)


def test_search_key_fixture(ref_data):
  say('search_key: reference fixture')
  d = np.load(os.path.join(ref_data, 'search_key.npz'))
  o = merged_octree(ref_data)
  xyzb = torch.from_numpy(d['xyzb']).to(DEV)
  key = xyz2key(xyzb[:, 0], xyzb[:, 1], xyzb[:, 2], xyzb[:, 3], 5)
  assert np.array_equal(np_(o.search_key(key, 5, False)), d['idx'])
  assert np.array_equal(np_(o.search_key(key, 5, True)), d['idx_ne'])
  assert np.array_equal(np_(o.search_xyzb(xyzb, 5, False)), d['idx'])
  assert np.array_equal(np_(o.search_xyzb(xyzb, 5, True)), d['idx_ne'])
  # the same queries through the walk down the tree (ocnn_locate_points), which the point
  # interpolation uses in place of the key search
  from ocnn_amd import _lib
  from ocnn_amd.nn.octree_interp import _tree
  pts = xyzb.float().contiguous()
  for ne, want in ((False, d['idx']), (True, d['idx_ne'])):
    got = torch.empty(pts.shape[0], dtype=torch.int32, device=DEV)
    _lib.check(_lib.lib().ocnn_locate_points(_lib.ptr(pts), pts.shape[0], *_tree(o, 5, ne), 0, _lib.ptr(got),
                                             _lib.stream()))
    assert np.array_equal(np_(got), want), ne


def test_octree_grow_split(ref_data):
  say('grow/split: regrow from the split masks')
  d = np.load(os.path.join(ref_data, 'batch_45.npz'))
  gt = merged_octree(ref_data)
  depth, full_depth = 6, 3
  o = Octree(depth, full_depth, batch_size=2, device=DEV)
  for dd in range(full_depth + 1):
    o.octree_grow_full(depth=dd)
  for dd in range(full_depth, depth + 1):
    o.octree_split((gt.children[dd] >= 0).long(), dd)
    if dd < depth:
      o.octree_grow(dd + 1)
  o.normals[depth] = gt.normals[depth]
  check_against(o, d)
  assert np.array_equal(np_(torch.cat(o.neighs[1:], dim=0)), d['neigh'])


def test_out_of_range_points_wrap():
  say('build: points outside [-1,1) wrap like the reference')
  pts = np.array([[1.0, 0.5, -0.25], [-1.01, 0.0, 0.0], [0.3, 1.2, -1.0], [0.999, -0.999, 0.1]],
                 np.float32)
  nrm = np.tile(np.array([[0, 0, 1]], np.float32), (4, 1))
  o = Octree(6, 2)
  idx = o.build_octree(Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV)))
  w, widx = R.build_octree(pts, nrm, depth=6, full_depth=2)
  assert np.array_equal(np_(torch.cat(o.keys)), np.concatenate(w.keys))
  assert np.array_equal(np_(torch.cat(o.children)), np.concatenate(w.children))
  assert np.array_equal(np_(idx), widx)


def test_bbox_arguments(ref_data):
  say('build: tensor bbmin/bbmax')
  d = np.load(os.path.join(ref_data, 'octree/test_002.npz'))
  lo = np.array([-1.1, -1.0, -1.2], np.float32)
  hi = np.array([1.0, 1.3, 1.0], np.float32)
  o = Octree(6, 2)
  o.build_octree(Points(torch.from_numpy(d['points']).to(DEV), torch.from_numpy(d['normals']).to(DEV)),
                 bbmin=torch.from_numpy(lo).to(DEV), bbmax=torch.from_numpy(hi).to(DEV))
  w, _ = R.build_octree(d['points'], d['normals'], depth=6, full_depth=2, bbmin=lo, bbmax=hi)
  assert np.array_equal(np_(torch.cat(o.keys)), np.concatenate(w.keys))
  assert np.array_equal(np_(torch.cat(o.children)), np.concatenate(w.children))


def test_larger_synthetic_batch_vs_oracle():
  say('build+neigh: 4 clouds x 30k points, depth 7, vs oracle')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 4, 7, n=30000)
  fea = torch.randn(pts.shape[0], 5, generator=torch.Generator().manual_seed(3))
  pc = Points(pts.to(DEV), nrm.to(DEV), fea.to(DEV), batch_id=bid.to(DEV), batch_size=4)
  o = Octree(7, 2, batch_size=4)
  idx = o.build_octree(pc)
  o.construct_all_neigh()
  w, widx = R.build_octree(pts.numpy(), nrm.numpy(), fea.numpy(), bid.numpy(), 7, 2, 4)
  R.construct_all_neigh(w)
  assert np.array_equal(o.nnum.numpy(), w.nnum) and np.array_equal(o.nnum_nempty.numpy(), w.nnum_nempty)
  for d in range(8):
    assert np.array_equal(np_(o.keys[d]), w.keys[d]), d
    assert np.array_equal(np_(o.children[d]), w.children[d]), d
    if d:
      assert np.array_equal(np_(o.neighs[d]), w.neighs[d]), d
  assert np.array_equal(np_(idx), widx)
  assert np.array_equal(np_(o.points[7]), w.points[7])
  assert np.array_equal(np_(o.features[7]), w.features[7])
  assert np.allclose(np_(o.normals[7]), w.normals[7], atol=1e-6)
  for kern, stride, ne in [('333', 1, True), ('222', 2, False), ('222', 2, True), ('333', 2, True)]:
    assert np.array_equal(np_(o._table(7, kern, stride, ne)), w.get_neigh(7, kern, stride, ne))


def test_full_size_invariants():
  say('build+neigh at the benchmark size: 8 x 100k points, depth 8 (properties only)')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 8, 1001, n=100000)
  pc = Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=8)
  o = Octree(8, 2, batch_size=8)
  idx = o.build_octree(pc)
  o.construct_all_neigh()
  assert int(idx.max()) + 1 == int(o.nnum_nempty[8])
  for d in range(3, 9):
    k = o.keys[d]
    assert bool((k[1:] > k[:-1]).all())                               # sorted, unique
    assert int(o.nnum[d]) == 8 * int(o.nnum_nempty[d - 1])
    c = o.children[d]
    assert torch.equal(c[c >= 0].long(), torch.arange(int(o.nnum_nempty[d]), device=DEV))
    t = o._table(d, '333', 1, False).long()
    n = t.shape[0]
    assert torch.equal(t[:, 13], torch.arange(n, device=DEV))          # centre slot = itself
    rows, slots = torch.nonzero(t >= 0, as_tuple=True)
    assert torch.equal(t[t[rows, slots], 26 - slots], rows)            # central symmetry
    # parent of every node holds it as a child: keys agree
    assert torch.equal(o.keys[d] >> 3 & ((1 << 45) - 1),
                       (o.keys[d - 1][o.nempty_index(d - 1)] & ((1 << 48) - 1)).repeat_interleave(8))
    t2 = o._table(d, '222', 2, False).long()
    assert torch.equal(t2, (torch.arange(n // 8, device=DEV) * 8).unsqueeze(1) +
                       torch.arange(8, device=DEV))
  # leaf of every point: its key is the leaf key
  leaf_key = o.keys[8][o.nempty_index(8)]
  p = (pts.to(DEV) + 1.0) * 128.0
  key = xyz2key(p[:, 0], p[:, 1], p[:, 2], bid.to(DEV).view(-1), 8)
  assert torch.equal(leaf_key[idx], key)


def test_random_octrees_vs_oracle():
  """Random depth / full depth / batch size / point counts (1 .. 40 000) and point
  distributions (uniform, a sphere, clusters with duplicates, grid-aligned coordinates up to the
  box faces): keys, children, counts, point -> leaf map, leaf signals and all neighbour tables
  bit exact against the oracle.  OCNN_TEST_CASES sets the number of cases (default 60)."""
  for case in random_cases(60):
    rng = np.random.default_rng(case)
    depth = int(rng.integers(2, 10))
    full = max(1, min(int(rng.integers(1, 5)), depth - 1))
    n = int(rng.choice([1, 2, 17, 500, 5000, 40000]))
    batch = min(int(rng.choice([1, 1, 2, 3, 5])), n)
    kind = int(rng.integers(0, 4))
    if kind == 0:
      pts = rng.uniform(-0.99, 0.99, (n, 3))
    elif kind == 1:
      v = rng.standard_normal((n, 3))
      pts = 0.9 * v / np.linalg.norm(v, axis=1, keepdims=True)
    elif kind == 2:
      c = rng.uniform(-0.8, 0.8, (5, 3))
      pts = c[rng.integers(0, 5, n)] + rng.normal(0, 0.01, (n, 3)) * (rng.random((n, 1)) < 0.7)
    else:
      pts = rng.integers(-2 ** depth // 2, 2 ** depth // 2, (n, 3)) / (2.0 ** (depth - 1))
    pts = np.clip(pts, -1.0, 0.999999).astype(np.float32)
    nrm = rng.standard_normal((n, 3)).astype(np.float32)
    fea = rng.standard_normal((n, 2)).astype(np.float32) if rng.random() < 0.5 else None
    bid = None
    if batch > 1:
      bid = rng.integers(0, batch, n)
      bid[:batch] = np.arange(batch)                         # every element has a point
      bid = np.sort(bid).astype(np.int64)
    say('random octree', case, 'depth', depth, 'full', full, 'batch', batch, 'points', n, 'kind', kind)
    pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV),
                None if fea is None else torch.from_numpy(fea).to(DEV),
                batch_id=None if bid is None else torch.from_numpy(bid).view(-1, 1).to(DEV), batch_size=batch)
    o = Octree(depth, full, batch_size=batch)
    idx = o.build_octree(pc)
    o.construct_all_neigh()
    w, widx = R.build_octree(pts, nrm, fea, bid, depth, full, batch)
    R.construct_all_neigh(w)
    assert np.array_equal(o.nnum.numpy(), w.nnum) and np.array_equal(o.nnum_nempty.numpy(), w.nnum_nempty)
    assert np.array_equal(np_(idx), widx)
    for d in range(depth + 1):
      assert np.array_equal(np_(o.keys[d]), w.keys[d]), d
      assert np.array_equal(np_(o.children[d]), w.children[d]), d
      if d:
        assert np.array_equal(np_(o.neighs[d]), w.neighs[d]), d
    assert np.array_equal(np_(o.points[depth]), w.points[depth])
    if fea is not None:
      assert np.array_equal(np_(o.features[depth]), w.features[depth])
    assert np.allclose(np_(o.normals[depth]), w.normals[depth], atol=1e-6)
    for kern, stride, ne in [('333', 1, True), ('222', 2, False), ('222', 2, True), ('333', 2, True),
                             ('313', 1, False), ('131', 2, True)]:
      assert np.array_equal(np_(o._table(depth, kern, stride, ne)), w.get_neigh(depth, kern, stride, ne))


@pytest.mark.parametrize('depth,full,batch,n', [(11, 2, 1, 3000), (11, 1, 5, 4000), (12, 3, 3, 2500),
                                                (10, 1, 2, 6000), (10, 2, 8, 6000), (16, 6, 1, 300),
                                                (3, 3, 2, 500), (2, 2, 1, 50), (4, 3, 3, 2000)])
def test_deep_octrees_vs_oracle(depth, full, batch, n):
  """Depths at which batch id and Morton code pass 32 bits (the build then sorts 64-bit keys),
  more than seven sparse layers (sixteen counters a point instead of eight), and octrees with no or
  one sparse layer (depth = full_depth, full_depth + 1): every layer's keys and children, the
  counts, the point -> leaf map and the leaf signals bit exact against the oracle."""
  say('deep octree: depth', depth, 'full', full, 'batch', batch, 'points', n)
  rng = np.random.default_rng(depth * 100 + batch)
  c = rng.uniform(-0.8, 0.8, (7, 3))
  pts = c[rng.integers(0, 7, n)] + rng.normal(0, 0.02, (n, 3)) * (rng.random((n, 1)) < 0.8)
  pts = np.clip(pts, -1.0, 0.999999).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32)
  bid = None
  if batch > 1:
    bid = rng.integers(0, batch, n)
    bid[:batch] = np.arange(batch)
    bid = np.sort(bid).astype(np.int64)
  pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV),
              batch_id=None if bid is None else torch.from_numpy(bid).view(-1, 1).to(DEV), batch_size=batch)
  o = Octree(depth, full, batch_size=batch)
  idx = o.build_octree(pc)
  w, widx = R.build_octree(pts, nrm, None, bid, depth, full, batch)
  assert np.array_equal(o.nnum.numpy(), w.nnum) and np.array_equal(o.nnum_nempty.numpy(), w.nnum_nempty)
  assert np.array_equal(np_(idx), widx)
  for d in range(depth + 1):
    assert np.array_equal(np_(o.keys[d]), w.keys[d]), d
    assert np.array_equal(np_(o.children[d]), w.children[d]), d
  assert np.array_equal(np_(o.points[depth]), w.points[depth])
  assert np.allclose(np_(o.normals[depth]), w.normals[depth], atol=1e-6)
  if depth <= 12:                                     # the tables too (one call for all layers)
    o.construct_all_neigh()
    R.construct_all_neigh(w)
    for d in range(1, depth + 1):
      assert np.array_equal(np_(o.neighs[d]), w.neighs[d]), d
      assert np.array_equal(np_(o.nempty_index(d)), np.nonzero(w.children[d] >= 0)[0]), d


def test_octree_without_a_full_layer_below_the_root():
  """full_depth = 0: the build equals the oracle's; the neighbour tables cannot be made (layer 1
  would need the table of layer 0, which does not exist - the reference's construct_neigh(1) fails
  on it too) and both routes refuse with an error instead of launching anything."""
  rng = np.random.default_rng(3)
  n, depth, batch = 400, 5, 2
  pts = rng.uniform(-0.9, 0.9, (n, 3)).astype(np.float32)
  nrm = rng.standard_normal((n, 3)).astype(np.float32)
  bid = np.sort(np.r_[0, 1, rng.integers(0, batch, n - 2)]).astype(np.int64)
  say('octree with full_depth 0')
  pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV),
              batch_id=torch.from_numpy(bid).view(-1, 1).to(DEV), batch_size=batch)
  o = Octree(depth, 0, batch_size=batch)
  idx = o.build_octree(pc)
  w, widx = R.build_octree(pts, nrm, None, bid, depth, 0, batch)
  assert np.array_equal(o.nnum.numpy(), w.nnum) and np.array_equal(o.nnum_nempty.numpy(), w.nnum_nempty)
  assert np.array_equal(np_(idx), widx)
  for d in range(depth + 1):
    assert np.array_equal(np_(o.keys[d]), w.keys[d]), d
    assert np.array_equal(np_(o.children[d]), w.children[d]), d
  with pytest.raises(AssertionError):
    o.construct_all_neigh()
  with pytest.raises(AssertionError):
    o.construct_neigh(1)
  with pytest.raises(TypeError):
    R.construct_all_neigh(w)


@pytest.mark.parametrize('depth,batch', [(8, 1), (9, 4), (6, 2)])
def test_uneven_clouds_vs_oracle(depth, batch):
  """Nine points in ten of a cloud inside one small cell (thousands of points to a leaf, a few
  leaves holding most of the cloud), next to an even cloud of the same size: both bit exact
  against the oracle."""
  n = 40000
  rng = np.random.default_rng(depth)
  for uneven in (True, False):
    say('uneven cloud' if uneven else 'even cloud', 'depth', depth, 'batch', batch)
    pts = rng.uniform(-0.95, 0.95, (n, 3))
    if uneven:
      pts[: 9 * n // 10] = np.array([0.3, -0.2, 0.6]) + rng.normal(0, 2e-4, (9 * n // 10, 3))
      pts = pts[rng.permutation(n)]
    pts = pts.astype(np.float32)
    nrm = rng.standard_normal((n, 3)).astype(np.float32)
    bid = None
    if batch > 1:
      bid = np.sort(rng.integers(0, batch, n)).astype(np.int64)
      bid[:batch] = np.arange(batch)
      bid = np.sort(bid)
    pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV),
                batch_id=None if bid is None else torch.from_numpy(bid).view(-1, 1).to(DEV), batch_size=batch)
    o = Octree(depth, 2, batch_size=batch)
    idx = o.build_octree(pc)
    w, widx = R.build_octree(pts, nrm, None, bid, depth, 2, batch)
    assert np.array_equal(o.nnum.numpy(), w.nnum) and np.array_equal(o.nnum_nempty.numpy(), w.nnum_nempty)
    assert np.array_equal(np_(idx), widx)
    for d in range(depth + 1):
      assert np.array_equal(np_(o.keys[d]), w.keys[d]), d
      assert np.array_equal(np_(o.children[d]), w.children[d]), d
    assert np.array_equal(np_(o.points[depth]), w.points[depth])
    assert np.allclose(np_(o.normals[depth]), w.normals[depth], atol=1e-6)


def test_input_feature_vs_oracle():
  """Octree.get_input_feature (ocnn/octree/octree.py:525-568) and modules.InputFeature: every
  letter and combinations, all nodes (zero rows for empty leaves) and non-empty nodes; the
  pieces are closed forms of the leaf signals: D = <L, N>, P = points / 2^(depth - 1) - 1."""
  from ocnn_amd.modules import InputFeature
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 3, 21, n=20000)
  fea = torch.randn(pts.shape[0], 4, generator=torch.Generator().manual_seed(2))
  o = Octree(6, 2, batch_size=3)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), fea.to(DEV), batch_id=bid.to(DEV), batch_size=3))
  w, _ = R.build_octree(pts.numpy(), nrm.numpy(), fea.numpy(), bid.numpy(), 6, 2, 3)
  for feature in ['N', 'D', 'L', 'P', 'F', 'ND', 'NDF', 'lpf', 'FPLDN']:
    for ne in (False, True):
      say('input feature', feature, 'nempty', ne)
      got = np_(o.get_input_feature(feature, ne))
      want = w.get_input_feature(feature, ne)
      assert got.shape == want.shape and got.dtype == np.float32
      assert np.abs(got - want).max() <= 2e-6, (feature, ne)
      assert np.array_equal(got, np_(InputFeature(feature, ne)(o)))
  nd = np_(o.get_input_feature('NDL', True))
  assert np.allclose(nd[:, 3], (nd[:, 4:7] * nd[:, 0:3]).sum(1), atol=1e-6)     # D = <L, N>
  assert np.abs(nd[:, 4:7]).max() <= 0.5
  empty = np_(o.children[6]) < 0
  assert not np_(o.get_input_feature('ND', False))[empty].any()
  # to_points: the leaf signals back as a point cloud in [-1, 1]
  back = o.to_points()
  assert np.allclose(np_(back.points), w.points[6] * 2.0 ** (1 - 6) - 1.0, atol=1e-6)
  assert np.array_equal(np_(back.normals), np_(o.normals[6]))


def test_random_octrees_regrown_from_split_masks():
  """octree_grow_full / octree_split / octree_grow (ocnn/octree/octree.py:289-402), as a
  generative decoder drives them: an octree regrown level by level from the split masks of a
  built one has the same keys, children, counts and neighbour tables (the property the
  reference's own test checks on its one file), on 25 random octrees (OCNN_TEST_CASES: another number)."""
  for case in random_cases(25):
    rng = np.random.default_rng(1000 + case)
    depth = int(rng.integers(3, 8))
    full = max(1, min(int(rng.integers(1, 4)), depth - 1))
    n = int(rng.choice([3, 40, 3000, 30000]))
    batch = min(int(rng.choice([1, 2, 3])), n)
    v = rng.standard_normal((n, 3))
    pts = (rng.uniform(0.2, 0.9) * v / np.linalg.norm(v, axis=1, keepdims=True)).astype(np.float32)
    bid = None
    if batch > 1:
      bid = rng.integers(0, batch, n)
      bid[:batch] = np.arange(batch)
      bid = np.sort(bid).astype(np.int64)
    say('regrow', case, 'depth', depth, 'full', full, 'batch', batch, 'points', n)
    built = Octree(depth, full, batch_size=batch)
    built.build_octree(Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(v.astype(np.float32)).to(DEV),
                              batch_id=None if bid is None else torch.from_numpy(bid).view(-1, 1).to(DEV),
                              batch_size=batch))
    built.construct_all_neigh()
    o = Octree(depth, full, batch_size=batch, device=DEV)
    for d in range(full + 1):
      o.octree_grow_full(depth=d)
    for d in range(full, depth + 1):
      o.octree_split((built.children[d] >= 0).long(), d)
      if d < depth:
        o.octree_grow(d + 1)
    assert np.array_equal(o.nnum.numpy(), built.nnum.numpy())
    assert np.array_equal(o.nnum_nempty.numpy(), built.nnum_nempty.numpy())
    for d in range(depth + 1):
      assert np.array_equal(np_(o.keys[d]), np_(built.keys[d])), d
      assert np.array_equal(np_(o.children[d]), np_(built.children[d])), d
      if d:
        assert np.array_equal(np_(o.neighs[d]), np_(built.neighs[d])), d


def test_random_merge_equals_batched_build():
  """merge_octrees of separately built octrees == build_octree on the merged cloud with batch
  ids (the identity the reference's test_octree.py:115-123 checks on its two files), on random
  clouds of unequal sizes: keys, children, counts, leaf signals, neighbour tables, batch_nnum
  (12 cases, or OCNN_TEST_CASES)."""
  for case in random_cases(12):
    rng = np.random.default_rng(2000 + case)
    depth = int(rng.integers(3, 8))
    full = max(1, min(int(rng.integers(1, 4)), depth - 1))
    batch = int(rng.integers(2, 5))
    clouds = []
    for b in range(batch):
      n = int(rng.choice([1, 30, 2000, 15000]))
      c = rng.uniform(-0.5, 0.5, 3)
      v = rng.standard_normal((n, 3))
      pts = np.clip(c + rng.uniform(0.1, 0.4) * v / np.linalg.norm(v, axis=1, keepdims=True), -0.99, 0.99)
      clouds.append((pts.astype(np.float32), v.astype(np.float32), rng.standard_normal((n, 2)).astype(np.float32)))
    say('merge', case, 'depth', depth, 'full', full, 'sizes', [len(c[0]) for c in clouds])
    singles, parts = [], []
    for pts, nrm, fea in clouds:
      pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV), torch.from_numpy(fea).to(DEV))
      parts.append(pc)
      o = Octree(depth, full)
      o.build_octree(pc)
      singles.append(o)
    merged = merge_octrees(singles)
    merged.construct_all_neigh()
    whole = Octree(depth, full, batch_size=batch)
    whole.build_octree(merge_points(parts))
    whole.construct_all_neigh()
    assert np.array_equal(merged.nnum.numpy(), whole.nnum.numpy())
    assert np.array_equal(merged.nnum_nempty.numpy(), whole.nnum_nempty.numpy())
    assert merged.batch_nnum.sum(1).tolist() == merged.nnum.tolist()
    assert merged.batch_nnum_nempty.sum(1).tolist() == merged.nnum_nempty.tolist()
    for d in range(depth + 1):
      assert np.array_equal(np_(merged.keys[d]), np_(whole.keys[d])), d
      assert np.array_equal(np_(merged.children[d]), np_(whole.children[d])), d
      if d:
        assert np.array_equal(np_(merged.neighs[d]), np_(whole.neighs[d])), d
    for name in ('points', 'normals', 'features'):
      assert np.array_equal(np_(getattr(merged, name)[depth]), np_(getattr(whole, name)[depth])), name


def test_octree_with_a_table_of_more_than_a_billion_entries():
  """8 x 1.1 M points at depth 11: 50 M nodes in the deepest layer, 1.35 G table entries (the
  library takes tables of up to 2^31).  Too large for the oracle; what must hold of any octree
  holds: keys sorted and unique per layer, eight children per non-empty parent, children
  numbered in order, the centre slot of every row is the row, central symmetry of the tables
  (the first and last 100 000 rows and 400 000 random ones per layer), and every point's leaf
  carries the point's key."""
  from ocnn_amd import synthetic
  depth = 11
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 8, 77, n=1100000)
  o = Octree(depth, 2, batch_size=8)
  idx = o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=8))
  o.construct_all_neigh()
  say('large octree: nodes per layer', o.nnum.tolist())
  assert int(o.nnum[depth]) * 27 > 1 << 30
  g = torch.Generator(device=DEV).manual_seed(3)
  for d in range(3, depth + 1):
    k = o.keys[d]
    assert bool((k[1:] > k[:-1]).all())
    assert int(o.nnum[d]) == 8 * int(o.nnum_nempty[d - 1])
    c = o.children[d]
    assert torch.equal(c[c >= 0].long(), torch.arange(int(o.nnum_nempty[d]), device=DEV))
    t = o._table(d, '333', 1, False)
    rows = t.shape[0]
    assert torch.equal(t[:, 13], torch.arange(rows, device=DEV, dtype=torch.int32))
    sel = torch.cat([torch.arange(0, min(rows, 100000), device=DEV), torch.arange(max(0, rows - 100000), rows, device=DEV),
                     torch.randint(0, rows, (400000,), device=DEV, generator=g)])
    ts = t[sel].long()
    at, slot = torch.nonzero(ts >= 0, as_tuple=True)
    assert torch.equal(t[ts[at, slot], 26 - slot].long(), sel[at]), d
    assert torch.equal(k >> 3 & ((1 << 45) - 1),
                       (o.keys[d - 1][o.nempty_index(d - 1)] & ((1 << 48) - 1)).repeat_interleave(8))
  leaf_key = o.keys[depth][o.nempty_index(depth)]
  p = (pts.to(DEV) + 1.0) * float(2 ** (depth - 1))
  assert torch.equal(leaf_key[idx], xyz2key(p[:, 0], p[:, 1], p[:, 2], bid.to(DEV).view(-1), depth))
  # one layer further the table would pass 2^31 entries: refused, not truncated
  big = Octree(depth + 1, 2, batch_size=8)
  big.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=8))
  if int(big.nnum[depth + 1]) * 27 >= 1 << 31:
    with pytest.raises(Exception):
      big.construct_all_neigh()

