"""GPU parity of key search, point interpolation, upsampling and max pooling: the HIP path
(through the C ABI) against the reference's data files and the numpy oracle."""

import os
import sys

import numpy as np
import pytest
from conftest import random_cases
import torch

import ocnn_amd
from ocnn_amd import synthetic
from ocnn_amd.nn import (octree_depad, octree_linear_pts, octree_max_pool, octree_max_unpool,
                         octree_nearest_pts, octree_nearest_upsample, OctreeInterp, OctreeMaxPool,
                         OctreeMaxUnpool, OctreeUpsample)
from ocnn_amd.octree import Octree, Points
from oracle import interp_ref as I
from test_gpu_octree import merged_octree, oracle_batch

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = {torch.float32: 1e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def np_(t):
  return t.detach().float().cpu().numpy() if t.is_floating_point() else t.detach().cpu().numpy()


def test_interp_against_reference_fixture(ref_data):
  """test/test_octree_interp.py:21-43 through the HIP path, with the reference's tolerance."""
  say('interp: reference fixture')
  t = np.load(os.path.join(ref_data, 'interp.npz'))
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  depth = 5
  data = torch.from_numpy(t['data']).to(DEV)
  pts = torch.from_numpy(t['pts']).to(DEV)
  data_ne = octree_depad(data, o, depth)
  got = {'linear': octree_linear_pts(data, o, depth, pts, nempty=False),
         'linear_ne': octree_linear_pts(data_ne, o, depth, pts, nempty=True),
         'near': octree_nearest_pts(data, o, depth, pts, nempty=False),
         'near_ne': octree_nearest_pts(data_ne, o, depth, pts, nempty=True)}
  for k, v in got.items():
    assert np.allclose(np_(v), t[k], atol=1e-6), k
  # and the oracle, also with the bounds check on points pushed out of the volume
  far = t['pts'].copy()
  far[::3, 1] -= 40.0
  for ne in (False, True):
    d = t['data'] if not ne else I.octree_depad(w, t['data'], depth)
    dg = data_ne if ne else data
    for bc in (False, True):
      fg = torch.from_numpy(far).to(DEV)
      assert np.allclose(np_(octree_linear_pts(dg, o, depth, fg, ne, bc)), I.linear_pts(w, d, depth, far, ne, bc), atol=1e-6)
      assert np.array_equal(np_(octree_nearest_pts(dg, o, depth, fg, ne, bc)), I.nearest_pts(w, d, depth, far, ne, bc))


@pytest.mark.parametrize('nempty', [False, True])
def test_nearest_upsample_and_modules(ref_data, nempty):
  """test/test_octree_interp.py:45-73, and the module forms against the oracle."""
  say('upsample', nempty)
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  depth = 4
  rows = int(o.nnum_nempty[depth] if nempty else o.nnum[depth])
  data = torch.rand(rows, 4, generator=torch.Generator().manual_seed(1)).to(DEV)
  out = octree_nearest_upsample(data, o, depth, nempty)
  xyzb = o.xyzb(depth + 1, nempty)
  pts = torch.stack(xyzb, dim=1).float()
  pts[:, :3] = (pts[:, :3] + 0.5) * 0.5
  ref = octree_nearest_pts(data, o, depth, pts, nempty, bound_check=True)
  assert torch.equal(out, ref)
  assert np.array_equal(np_(out), I.nearest_upsample(w, np_(data), depth, nempty))
  assert torch.equal(OctreeUpsample('nearest', nempty)(data, o, depth), out)
  for target in (depth + 1, depth + 2):
    got = OctreeUpsample('linear', nempty)(data, o, depth, target)
    assert np.allclose(np_(got), I.upsample(w, np_(data), depth, target, 'linear', nempty), atol=1e-6)
    got = OctreeUpsample('nearest', nempty)(data, o, depth, target)
    assert np.array_equal(np_(got), I.upsample(w, np_(data), depth, target, 'nearest', nempty))
  assert OctreeUpsample('linear', nempty)(data, o, depth, depth) is data
  # OctreeInterp rescales the points from the bounding box in place
  p = (torch.rand(300, 4, generator=torch.Generator().manual_seed(2)) * 2 - 1)
  p[:, 3] = (p[:, 3] > 0).float()
  pg = p.clone().to(DEV)
  got = OctreeInterp('linear', nempty, bound_check=True)(data, o, depth, pg)
  scaled = p.numpy().copy()
  scaled[:, :3] = (scaled[:, :3] + 1.0) * (2 ** depth / 2.0)
  assert np.allclose(np_(pg), scaled, atol=1e-6)
  assert np.allclose(np_(got), I.linear_pts(w, np_(data), depth, scaled, nempty, True), atol=1e-6)


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_interp_gradients_and_dtypes(ref_data, dtype):
  """Gradient with respect to the data (the transposed sparse product, no atomics): against
  the oracle, and the same bits on a second run; 16-bit data against the fp32 definition."""
  say('interp gradients', dtype)
  t = np.load(os.path.join(ref_data, 'interp.npz'))
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  depth = 5
  g = torch.Generator().manual_seed(3)
  for ne in (False, True):
    rows = int(o.nnum_nempty[depth] if ne else o.nnum[depth])
    pts = torch.from_numpy(t['pts']).to(DEV)
    data = torch.randn(rows, 8, generator=g).to(dtype).to(DEV).requires_grad_()
    grad = torch.randn(pts.shape[0], 8, generator=g).to(dtype).to(DEV)
    out = octree_linear_pts(data, o, depth, pts, ne)
    assert out.dtype == dtype
    want = I.linear_pts(w, np_(data), depth, t['pts'], ne)
    assert np.abs(np_(out) - want).max() <= TOL[dtype] * max(1.0, np.abs(want).max())
    out.backward(grad)
    gd = data.grad.clone()
    wantg = I.linear_pts_grad(w, np_(grad), depth, t['pts'], rows, ne)
    assert np.abs(np_(gd) - wantg).max() <= max(TOL[dtype], 1e-5) * max(1.0, np.abs(wantg).max())
    data.grad = None
    octree_linear_pts(data, o, depth, pts, ne).backward(grad)
    assert torch.equal(data.grad, gd)
    # nearest: every point passes its gradient to the one row it read
    data.grad = None
    octree_nearest_pts(data, o, depth, pts, ne).backward(grad)
    idx = I.search_xyzb(w, t['pts'], depth, ne)
    wantn = np.zeros((rows, 8))
    np.add.at(wantn, idx[idx >= 0], np_(grad).astype(np.float64)[idx >= 0])
    assert np.abs(np_(data.grad) - wantn).max() <= max(TOL[dtype], 1e-5) * max(1.0, np.abs(wantn).max())


@pytest.mark.parametrize('nempty', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_max_pool_unpool_vs_oracle(ref_data, nempty, dtype):
  """octree_max_pool / octree_max_unpool and their gradients, depths with full and sparse
  parents, against the oracle (values are copies: exact in every dtype)."""
  say('max pool', nempty, dtype)
  o = merged_octree(ref_data)
  w = oracle_batch(ref_data)
  g = torch.Generator().manual_seed(4)
  for depth in (3, 4, 6):
    rows = int(o.nnum_nempty[depth] if nempty else o.nnum[depth])
    data = torch.randn(rows, 5, generator=g).to(dtype)
    dg = data.to(DEV).requires_grad_()
    out, idx = octree_max_pool(dg, o, depth, nempty, return_indices=True)
    want, widx = I.max_pool(w, data.float().numpy(), depth, nempty)
    assert np.array_equal(np_(out), want) and np.array_equal(np_(idx), widx)
    assert idx.dtype == torch.long
    assert torch.equal(OctreeMaxPool(nempty)(dg, o, depth), out)
    # gradient of pooling = unpooling of the gradient
    grad = torch.randn(out.shape, generator=g).to(dtype)
    out.backward(grad.to(DEV))
    assert np.array_equal(np_(dg.grad), I.max_unpool(w, grad.float().numpy(), widx, depth - 1, nempty))
    # unpooling, module form, and its gradient (a gather at the indices)
    pooled = out.detach().clone().requires_grad_()
    up = OctreeMaxUnpool(nempty)(pooled, idx, o, depth - 1)
    assert np.array_equal(np_(up), I.max_unpool(w, want, widx, depth - 1, nempty))
    gu = torch.randn(up.shape, generator=g).to(dtype)
    up.backward(gu.to(DEV))
    full = gu.float().numpy() if not nempty else I.octree_pad(w, gu.float().numpy(), depth)
    picked = np.take_along_axis(full.reshape(-1, 8, 5), widx[:, None, :], 1)[:, 0]
    wantg = picked if nempty else I.octree_pad(w, picked, depth - 1)
    assert np.array_equal(np_(pooled.grad), wantg)


def test_interp_and_pool_at_full_size():
  """The benchmark octree (8 x 100k points, depth 8): properties that need no oracle run.
  A constant field interpolates to the constant wherever a neighbour exists; interpolating
  at the node centres returns the node values; nearest upsampling followed by max pooling
  is the identity on non-empty nodes; pooling picks a value that is present."""
  say('interp / pool: full size')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 8, 1001, n=100000)
  o = Octree(8, 2, batch_size=8)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=8))
  depth = 8
  rows = int(o.nnum_nempty[depth])
  q = torch.cat([(pts.to(DEV) + 1.0) * 128.0, bid.to(DEV).float().view(-1, 1)], 1)
  const = torch.full((rows, 3), 2.5, device=DEV)
  out = octree_linear_pts(const, o, depth, q, nempty=True)
  assert torch.allclose(out, torch.full_like(out, 2.5), atol=1e-5)          # every point lies in a leaf
  near = octree_nearest_pts(const, o, depth, q, nempty=True)
  assert bool((near == 2.5).all())
  data = torch.randn(rows, 16, generator=torch.Generator().manual_seed(6)).to(DEV)
  x, y, z, b = o.xyzb(depth, nempty=True)
  centres = torch.stack([x + 0.5, y + 0.5, z + 0.5, b], 1).float()
  assert torch.equal(octree_nearest_pts(data, o, depth, centres, nempty=True), data)
  assert torch.allclose(octree_linear_pts(data, o, depth, centres, nempty=True), data, atol=1e-5)
  coarse = torch.randn(int(o.nnum_nempty[depth - 1]), 16, generator=torch.Generator().manual_seed(7)).to(DEV)
  up = octree_nearest_upsample(coarse, o, depth - 1, nempty=True)
  assert torch.equal(octree_max_pool(up, o, depth, nempty=True), coarse)
  pooled, idx = octree_max_pool(data, o, depth, nempty=True, return_indices=True)
  back = octree_max_unpool(pooled, idx, o, depth - 1, nempty=True)
  hit = back != 0
  assert torch.equal(back[hit], data[hit])
  assert int(hit.sum()) == pooled.numel() - int((pooled == 0).sum())       # (a maximum may be exactly 0)


def _to_voxels(data, o, depth):
  x, y, z, b = o.xyzb(depth, False)
  n = 1 << depth
  vox = data.new_zeros([o.batch_size, n, n, n, data.shape[1]])
  vox[b, x, y, z] = data
  return vox


def test_avg_pool_is_avg_pool3d_on_a_full_layer(ref_data):
  """test/test_octree_pool.py:39-61: on a full layer the average over the existing neighbours
  is torch.nn.AvgPool3d without the padding counted; and the gradient is its adjoint."""
  from ocnn_amd.nn import OctreeAvgPool, octree_avg_pool
  say('avg pool')
  o = merged_octree(ref_data)
  depth, c = 3, 33
  data = torch.rand(int(o.nnum[depth]), c, generator=torch.Generator().manual_seed(8)).to(DEV)
  grid = _to_voxels(data, o, depth)
  for kernel, stride, pad in [(3, 1, 1), (3, 2, 1), (2, 2, 0)]:
    want = torch.nn.AvgPool3d(kernel, stride, pad, count_include_pad=False)(grid.permute(0, 4, 1, 2, 3)).permute(0, 2, 3, 4, 1)
    out = OctreeAvgPool([kernel], stride, nempty=False)(data, o, depth)
    got = _to_voxels(out, o, depth - 1 if stride == 2 else depth)
    assert torch.allclose(got, want, atol=1e-6), (kernel, stride)
  # sparse level, gradient: <pool(x), g> = <x, pool^T(g)>
  depth = 5
  x = torch.randn(int(o.nnum_nempty[depth]), 6, generator=torch.Generator().manual_seed(9)).to(DEV).requires_grad_()
  y = octree_avg_pool(x, o, depth, '333', 1, nempty=True)
  g = torch.randn(y.shape, generator=torch.Generator().manual_seed(10)).to(DEV)
  y.backward(g)
  t = o.get_neigh(depth, '333', 1, True)
  cnt = (t >= 0).sum(1).clamp(min=1).float()
  want = torch.zeros_like(x)
  for k in range(27):
    v = t[:, k] >= 0
    want.index_add_(0, t[v, k], g[v] / cnt[v, None])
  assert torch.allclose(x.grad, want, atol=1e-5)


@pytest.mark.parametrize('nempty', [False, True])
def test_global_pool(ref_data, nempty):
  from ocnn_amd.nn import OctreeGlobalPool
  say('global pool', nempty)
  o = merged_octree(ref_data)
  depth = 5
  rows = int(o.nnum_nempty[depth] if nempty else o.nnum[depth])
  x = torch.randn(rows, 7, generator=torch.Generator().manual_seed(12)).to(DEV).requires_grad_()
  out = OctreeGlobalPool(nempty)(x, o, depth)
  bid = o.batch_id(depth, nempty)
  assert out.shape == (2, 7)
  for b in range(2):
    assert torch.allclose(out[b], x.detach()[bid == b].mean(0), atol=1e-5)
  g = torch.randn(2, 7, generator=torch.Generator().manual_seed(13)).to(DEV)
  out.backward(g)
  cnt = torch.bincount(bid, minlength=2).float()
  assert torch.allclose(x.grad, (g / cnt[:, None])[bid], atol=1e-6)


def test_walk_down_the_tree_equals_the_key_search():
  """ocnn_locate_points / ocnn_interp_linear_locate (a node found by walking down from the
  deepest full layer) against ocnn_search_points / ocnn_interp_linear_prepare (binary search
  over the layer's keys, pinned by the reference's search fixture): the same rows, weights and
  weight sums, bit for bit, for points inside, on the faces of and outside the volume, batch ids
  that no octree has, every depth of two octrees (depths that are and are not multiples of 3,
  above and below the full depth), all nodes and non-empty ones, with and without the bounds check."""
  import ctypes
  from ocnn_amd import _lib
  L = _lib.lib()
  g = torch.Generator().manual_seed(23)
  for batch, depth_max, full in ((3, 7, 2), (1, 5, 3)):
    pts3, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, batch, 5, n=6000)
    o = Octree(depth_max, full, batch_size=batch)
    o.build_octree(Points(pts3.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV) if batch > 1 else None, batch_size=batch))
    for depth in range(1, depth_max + 1):
      scale = float(1 << depth)
      n = 5000
      q = torch.rand(n, 3, generator=g) * (scale + 4.0) - 2.0             # some outside on every side
      q[:500] = torch.randint(0, (1 << depth) + 1, (500, 3), generator=g).float()      # on cell faces and corners
      pick = torch.randint(0, pts3.shape[0], (2000,), generator=g)
      q[500:2500] = (pts3[pick] + 1.0) * scale / 2 + torch.randn(2000, 3, generator=g) * 0.7   # around the surface
      b = torch.randint(-1, batch + 2, (n, 1), generator=g).float()
      b[500:2500] = bid[pick].float().view(-1, 1) if batch > 1 else 0.0
      pts = torch.cat([q, b], 1).contiguous().to(DEV)
      for nempty in (False, True):
        keys = o.key(depth, nempty).contiguous()
        children = (ctypes.c_void_p * (depth + 1))(*[o.children[l].data_ptr() for l in range(depth + 1)])
        tree = (children, depth, full, batch, int(nempty))
        for check in (0, 1):
          say('walk down the tree', batch, depth, nempty, check)
          want = torch.empty(n, dtype=torch.int32, device=DEV)
          got = torch.empty(n, dtype=torch.int32, device=DEV)
          _lib.check(L.ocnn_search_points(_lib.ptr(pts), n, depth, _lib.ptr(keys), keys.numel(), check,
                                          _lib.ptr(want), _lib.stream()))
          _lib.check(L.ocnn_locate_points(_lib.ptr(pts), n, *tree, check, _lib.ptr(got), _lib.stream()))
          assert torch.equal(got, want)
          assert int((want >= 0).sum()) > 100
          outs = []
          for fn, args in ((L.ocnn_interp_linear_prepare, (depth, _lib.ptr(keys), keys.numel())),
                           (L.ocnn_interp_linear_locate, tree)):
            idx = torch.empty((n, 8), dtype=torch.int32, device=DEV)
            w = torch.empty((n, 8), dtype=torch.float32, device=DEV)
            norm = torch.empty(n, dtype=torch.float32, device=DEV)
            _lib.check(fn(_lib.ptr(pts), n, *args, check, _lib.ptr(idx), _lib.ptr(w), _lib.ptr(norm), _lib.stream()))
            outs.append((idx, w, norm))
          for a, c in zip(*outs):
            assert torch.equal(a, c)


def test_transposed_matrix_edge_cases():
  """ocnn_csr_transpose on matrices without any entry, with one point, with rows nobody reads and
  with every entry on one row: row pointers, columns in point order and values against a direct
  construction."""
  from ocnn_amd.nn.octree_interp import _transpose
  g = torch.Generator().manual_seed(2)
  for points, k, rows, mode in [(5, 8, 7, 'none'), (1, 8, 3, 'some'), (300, 8, 1000, 'some'), (300, 1, 4, 'one row'),
                                (2000, 8, 50, 'some')]:
    say('transposed matrix', points, k, rows, mode)
    if mode == 'none':
      idx = torch.full((points, k), -1, dtype=torch.int32)
    elif mode == 'one row':
      idx = torch.full((points, k), 2, dtype=torch.int32)
    else:
      idx = torch.randint(-1, rows, (points, k), generator=g, dtype=torch.int32)
    w = torch.rand(points, k, generator=g)
    norm = torch.rand(points, generator=g) + 0.5
    rowptr, col, val = _transpose(idx.to(DEV), w.to(DEV), norm.to(DEV), rows)
    rowptr, col, val = rowptr.cpu().numpy(), col.cpu().numpy(), val.cpu().numpy()
    flat = idx.numpy().reshape(-1)
    want_rows = [np.nonzero(flat == r)[0] for r in range(rows)]          # ascending entry = point order
    assert rowptr[0] == 0 and rowptr[-1] == sum(len(e) for e in want_rows)
    for r, e in enumerate(want_rows):
      assert rowptr[r + 1] - rowptr[r] == len(e), r
      assert np.array_equal(col[rowptr[r]:rowptr[r + 1]], e // k), r
      wantv = w.numpy().reshape(-1)[e] / (norm.numpy()[e // k] + np.float32(1e-12))
      assert np.allclose(val[rowptr[r]:rowptr[r + 1]], wantv, rtol=1e-6), r
    # without weights and norm: no values
    rowptr2, col2, val2 = _transpose(idx.to(DEV), None, None, rows)
    assert val2 is None and np.array_equal(rowptr2.cpu().numpy(), rowptr)
    assert np.array_equal(col2.cpu().numpy()[:rowptr[-1]], col[:rowptr[-1]])


def test_random_interp_and_pool_vs_oracle():
  """Random octrees (depth 2 .. 8, one to four clouds, 1 .. 10 000 points), a random layer of
  each, all or non-empty nodes, bounds check on or off, 1 .. 20 channels, 1 .. 5 000 query points
  scattered around the cloud with some beyond the volume on either side: trilinear and nearest
  interpolation, the gradient of the former, max pooling with its indices and nearest upsampling
  against the oracle.  OCNN_TEST_CASES sets the number of cases (default 60)."""
  from oracle import octree_ref as R
  for case in random_cases(60):
    rng = np.random.default_rng(9000 + case)
    depth = int(rng.integers(2, 9))
    full = max(1, min(int(rng.integers(1, 4)), depth))
    n = int(rng.choice([1, 5, 100, 2000, 10000]))
    batch = min(int(rng.choice([1, 1, 2, 4])), n)
    c = rng.uniform(-0.8, 0.8, (4, 3))
    pts = np.clip(c[rng.integers(0, 4, n)] + rng.normal(0, 0.15, (n, 3)), -1.0, 0.999999).astype(np.float32)
    nrm = rng.standard_normal((n, 3)).astype(np.float32)
    bid = None
    if batch > 1:
      bid = rng.integers(0, batch, n)
      bid[:batch] = np.arange(batch)
      bid = np.sort(bid).astype(np.int64)
    d = int(rng.integers(1, depth + 1))
    ne, bc = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    C = int(rng.choice([1, 3, 8, 16, 20]))
    m = int(rng.choice([1, 7, 300, 5000]))
    say('random interp', case, 'depth', depth, 'full', full, 'batch', batch, 'points', n, 'layer', d, 'nempty', ne,
        'bound check', bc, 'channels', C, 'queries', m)
    pc = Points(torch.from_numpy(pts).to(DEV), torch.from_numpy(nrm).to(DEV),
                batch_id=None if bid is None else torch.from_numpy(bid).view(-1, 1).to(DEV), batch_size=batch)
    o = Octree(depth, full, batch_size=batch)
    o.build_octree(pc)
    o.construct_all_neigh()
    w, _ = R.build_octree(pts, nrm, None, bid, depth, full, batch)
    R.construct_all_neigh(w)
    rows = int(o.nnum_nempty[d] if ne else o.nnum[d])
    data = rng.standard_normal((rows, C)).astype(np.float32)
    src = rng.integers(0, n, m)
    q = (pts[src] + 1.0) * 2.0 ** (d - 1) + rng.normal(0, 0.7, (m, 3))
    q[rng.random(m) < 0.05] -= 2.0 ** d
    q[rng.random(m) < 0.05] += 2.0 ** d
    qb = (bid[src] if bid is not None else np.zeros(m)).astype(np.float32)
    q = np.concatenate([q.astype(np.float32), qb[:, None]], 1)
    dg = torch.from_numpy(data).to(DEV).requires_grad_()
    qg = torch.from_numpy(q).to(DEV)
    out = octree_linear_pts(dg, o, d, qg.clone(), ne, bc)
    assert np.allclose(np_(out), I.linear_pts(w, data, d, q, ne, bc), atol=2e-5), case
    grad = rng.standard_normal((m, C)).astype(np.float32)
    out.backward(torch.from_numpy(grad).to(DEV))
    wantg = I.linear_pts_grad(w, grad, d, q, rows, ne, bc)
    assert np.allclose(np_(dg.grad), wantg, atol=2e-4 * max(1.0, np.abs(wantg).max())), case
    assert np.array_equal(np_(octree_nearest_pts(dg, o, d, qg.clone(), ne, bc)), I.nearest_pts(w, data, d, q, ne, bc)), case
    if d >= 2:
      po, pi = octree_max_pool(dg.detach(), o, d, ne, return_indices=True)
      wp, wi = I.max_pool(w, data, d, ne)
      assert np.array_equal(np_(po), wp) and np.array_equal(np_(pi), wi), case
    if d < depth:
      assert np.array_equal(np_(octree_nearest_upsample(dg.detach(), o, d, ne)), I.nearest_upsample(w, data, d, ne)), case
