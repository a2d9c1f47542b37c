"""Pins the conv / deconv / depth-wise conv oracle.  The reference's golden file
for conv values is absent from its checkout, so the pins are: library special
cases (dense conv3d on a full octree layer), spatial brute force through key
search, exact bilinear/adjoint identities and chunked-vs-unchunked agreement.
CPU only."""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import conv_ref as C
from oracle import octree_ref as R


@pytest.fixture(scope='module')
def oct(ref_data):
  d4 = np.load(os.path.join(ref_data, 'octree/test_004.npz'))
  d5 = np.load(os.path.join(ref_data, 'octree/test_005.npz'))
  pts = np.concatenate([d4['points'], d5['points']])
  nrm = np.concatenate([d4['normals'], d5['normals']])
  bid = np.concatenate([np.zeros(len(d4['points'])), np.ones(len(d5['points']))])
  o, _ = R.build_octree(pts, nrm, batch_id=bid, depth=6, full_depth=3, batch_size=2)
  R.construct_all_neigh(o)
  return o


def to_vox(o, data, depth):
  """vox[b, x, y, z, c] = data[row] (the reference's octree2voxel)."""
  x, y, z, b = R.key2xyz(o.keys[depth], depth)
  n = 1 << depth
  vox = np.zeros((o.batch_size, n, n, n, data.shape[1]), data.dtype)
  vox[b, x, y, z] = data
  return vox, (b, x, y, z)


def dense_weight(W, ks):
  """W (K, Cin, Cout) with slot order kx-major -> conv3d weight (Cout, Cin, kx, ky, kz)."""
  K, ci, co = W.shape
  return torch.from_numpy(W.reshape(ks[0], ks[1], ks[2], ci, co)).permute(4, 3, 0, 1, 2)


# ---- library special cases on a full layer ---------------------------------

@pytest.mark.parametrize('kernel', ['333', '311', '131', '113', '331', '313', '133'])
def test_full_layer_equals_conv3d(oct, kernel):
  d, ci, co = 3, 3, 5
  rng = np.random.default_rng(1)
  ks = [int(c) for c in kernel]
  K = ks[0] * ks[1] * ks[2]
  data = rng.standard_normal((int(oct.nnum[d]), ci))
  W = rng.standard_normal((K, ci, co))
  out = C.conv_layer(oct, data, W, d, ks, 1, False)
  vox, (b, x, y, z) = to_vox(oct, data, d)
  ref = F.conv3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), dense_weight(W, ks),
                 padding=[k // 2 for k in ks])
  ref = ref.permute(0, 2, 3, 4, 1).numpy()[b, x, y, z]
  assert np.allclose(out, ref, atol=1e-12)


def test_full_layer_stride2_equals_conv3d(oct):
  d, ci, co = 3, 4, 3
  rng = np.random.default_rng(2)
  data = rng.standard_normal((int(oct.nnum[d]), ci))
  W = rng.standard_normal((8, ci, co))
  out = C.conv_layer(oct, data, W, d, [2], 2, False)
  assert out.shape[0] == oct.nnum[d - 1]
  vox, _ = to_vox(oct, data, d)
  ref = F.conv3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), dense_weight(W, [2, 2, 2]),
                 stride=2).permute(0, 2, 3, 4, 1).numpy()
  x, y, z, b = R.key2xyz(oct.keys[d - 1], d - 1)
  assert np.allclose(out, ref[b, x, y, z], atol=1e-12)


def test_full_layer_stride2_333_equals_conv3d(oct):
  # 3x3x3 stride 2: window centred on the first sibling (offsets -1..1 around 2p)
  d, ci, co = 3, 2, 3
  rng = np.random.default_rng(3)
  data = rng.standard_normal((int(oct.nnum[d]), ci))
  W = rng.standard_normal((27, ci, co))
  out = C.conv_layer(oct, data, W, d, [3], 2, False)
  vox, _ = to_vox(oct, data, d)
  ref = F.conv3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), dense_weight(W, [3, 3, 3]),
                 stride=2, padding=1).permute(0, 2, 3, 4, 1).numpy()
  x, y, z, b = R.key2xyz(oct.keys[d - 1], d - 1)
  assert np.allclose(out, ref[b, x, y, z], atol=1e-12)


def test_full_layer_deconv_equals_conv_transpose3d(oct):
  d, ci, co = 2, 3, 4                       # depth 2 -> depth 3, both full
  rng = np.random.default_rng(4)
  data = rng.standard_normal((int(oct.nnum[d]), ci))
  W = rng.standard_normal((8, co, ci))      # deconv weights: (K, out_ch, in_ch)
  out = C.deconv_layer(oct, data, W, d, [2], 2, False)
  assert out.shape == (oct.nnum[d + 1], co)
  vox, _ = to_vox(oct, data, d)
  # conv_transpose3d weight: (in_ch, out_ch, kx, ky, kz)
  wt = torch.from_numpy(W.reshape(2, 2, 2, co, ci)).permute(4, 3, 0, 1, 2)
  ref = F.conv_transpose3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), wt, stride=2)
  ref = ref.permute(0, 2, 3, 4, 1).numpy()
  x, y, z, b = R.key2xyz(oct.keys[d + 1], d + 1)
  assert np.allclose(out, ref[b, x, y, z], atol=1e-12)


def test_full_layer_deconv_stride1_equals_conv_transpose3d(oct):
  d, ci, co = 3, 2, 3
  rng = np.random.default_rng(5)
  data = rng.standard_normal((int(oct.nnum[d]), ci))
  W = rng.standard_normal((27, co, ci))
  out = C.deconv_layer(oct, data, W, d, [3], 1, False)
  vox, (b, x, y, z) = to_vox(oct, data, d)
  wt = torch.from_numpy(W.reshape(3, 3, 3, co, ci)).permute(4, 3, 0, 1, 2)
  ref = F.conv_transpose3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), wt, padding=1)
  ref = ref.permute(0, 2, 3, 4, 1).numpy()[b, x, y, z]
  assert np.allclose(out, ref, atol=1e-12)


def test_full_layer_dwconv_equals_grouped_conv3d(oct):
  d, c = 3, 6
  rng = np.random.default_rng(6)
  data = rng.standard_normal((int(oct.nnum[d]), c))
  W = rng.standard_normal((27, 1, c))
  out = C.dwconv_layer(oct, data, W, d, [3], 1, False)
  vox, (b, x, y, z) = to_vox(oct, data, d)
  wd = torch.from_numpy(W.reshape(3, 3, 3, c)).permute(3, 0, 1, 2).unsqueeze(1)
  ref = F.conv3d(torch.from_numpy(vox).permute(0, 4, 1, 2, 3), wd, padding=1, groups=c)
  ref = ref.permute(0, 2, 3, 4, 1).numpy()[b, x, y, z]
  assert np.allclose(out, ref, atol=1e-12)


# ---- spatial brute force on sparse levels -----------------------------------

def spatial_conv(oct, data, W, depth, ks, stride, nempty):
  """Definition in space: output cell c (every node, or every non-empty node;
  for stride 2 every parent node) sums W[offset] * data[cell at base + offset]
  where the cell exists.  Pure Python over slots, key search for the cells."""
  din, dout = depth, depth - 1 if stride == 2 else depth
  key_in = oct.keys[din]
  if nempty:
    key_in = key_in[oct.nempty_index(din)]
  key_out = oct.keys[dout]
  if nempty or stride == 2:
    key_out = key_out[oct.nempty_index(dout)]
  x, y, z, b = R.key2xyz(key_out, dout)
  if stride == 2:
    x, y, z = 2 * x, 2 * y, 2 * z
  offs = [[0, 1] if k == 2 else ([0] if k == 1 else [-1, 0, 1]) for k in ks]
  out = np.zeros((len(key_out), W.shape[2]))
  n = 1 << din
  slot = 0
  for dx in offs[0]:
    for dy in offs[1]:
      for dz in offs[2]:
        xx, yy, zz = x + dx, y + dy, z + dz
        ok = (xx >= 0) & (yy >= 0) & (zz >= 0) & (xx < n) & (yy < n) & (zz < n)
        q = R.xyz2key(xx, yy, zz, b, din)
        pos = np.searchsorted(key_in, q)
        pos[pos >= len(key_in)] = 0
        hit = ok & (key_in[pos] == q)
        out[hit] += data[pos[hit]] @ W[slot]
        slot += 1
  return out


GRID = [(k, s, ne) for k in ['333', '222', '311', '131', '113', '331', '313', '133']
        for s in (1, 2) for ne in (False, True)]


@pytest.mark.parametrize('kernel,stride,nempty', GRID)
def test_conv_spatial_brute_force(oct, kernel, stride, nempty):
  d, ci, co = 5, 3, 2
  ks = [int(c) for c in kernel]
  rng = np.random.default_rng(7)
  rows = int(oct.nnum_nempty[d] if nempty else oct.nnum[d])
  data = rng.standard_normal((rows, ci))
  W = rng.standard_normal((ks[0] * ks[1] * ks[2], ci, co))
  out = C.conv_layer(oct, data, W, d, ks, stride, nempty)
  want = spatial_conv(oct, data, W, d, ks, stride, nempty)
  if stride == 2 and not nempty:
    want = C.octree_pad(want, oct, d - 1)
  assert out.shape == want.shape
  assert np.allclose(out, want, atol=1e-12)


# ---- exact identities -------------------------------------------------------

@pytest.mark.parametrize('kernel,stride,nempty', GRID)
def test_conv_adjoint_and_bilinear(oct, kernel, stride, nempty):
  d, ci, co = 5, 3, 4
  ks = [int(c) for c in kernel]
  K = ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(8)
  rows = int(oct.nnum_nempty[d] if nempty else oct.nnum[d])
  data = rng.standard_normal((rows, ci))
  W = rng.standard_normal((K, ci, co))
  out = C.conv_layer(oct, data, W, d, ks, stride, nempty)
  g = rng.standard_normal(out.shape)
  _, gx, gW, gb = C.conv_layer(oct, data, W, d, ks, stride, nempty, grad=g)
  lhs = (out * g).sum()
  assert np.isclose(lhs, (data * gx).sum(), rtol=1e-10)
  assert np.isclose(lhs, (W * gW).sum(), rtol=1e-10)


@pytest.mark.parametrize('kernel,stride,nempty', GRID)
def test_deconv_is_adjoint_of_conv(oct, kernel, stride, nempty):
  # OctreeDeconv(W) is the data-gradient of OctreeConv(W) (octree_conv.py:271,285)
  d, ci, co = 4, 2, 3                      # deconv input at depth d
  ks = [int(c) for c in kernel]
  K = ks[0] * ks[1] * ks[2]
  rng = np.random.default_rng(9)
  dd = d + 1 if stride == 2 else d         # the finer side
  rows = int(oct.nnum_nempty[d] if nempty else oct.nnum[d])
  data = rng.standard_normal((rows, ci))
  W = rng.standard_normal((K, co, ci))     # (K, deconv out, deconv in)
  out = C.deconv_layer(oct, data, W, d, ks, stride, nempty)
  fine_rows = int(oct.nnum_nempty[dd] if nempty else oct.nnum[dd])
  assert out.shape == (fine_rows, co)
  y = rng.standard_normal(out.shape)
  conv_y = C.conv_layer(oct, y, W, dd, ks, stride, nempty)   # co -> ci
  assert np.isclose((out * y).sum(), (data * conv_y).sum(), rtol=1e-10)
  _, gx, gW, _ = C.deconv_layer(oct, data, W, d, ks, stride, nempty, grad=y)
  assert np.isclose((out * y).sum(), (data * gx).sum(), rtol=1e-10)
  assert np.isclose((out * y).sum(), (W * gW).sum(), rtol=1e-10)


def test_dwconv_equals_per_channel_conv(oct):
  # the reference's own cross-check (test/test_octree_dwconv.py:18-55)
  d, c = 5, 5
  rng = np.random.default_rng(10)
  for kernel, stride, nempty in GRID[::3]:
    ks = [int(ch) for ch in kernel]
    K = ks[0] * ks[1] * ks[2]
    rows = int(oct.nnum_nempty[d] if nempty else oct.nnum[d])
    data = rng.standard_normal((rows, c))
    W = rng.standard_normal((K, 1, c))
    out = C.dwconv_layer(oct, data, W, d, ks, stride, nempty)
    g = rng.standard_normal(out.shape)
    _, gx, gW, _ = C.dwconv_layer(oct, data, W, d, ks, stride, nempty, grad=g)
    for ch in range(c):
      o1, gx1, gW1, _ = C.conv_layer(oct, data[:, ch:ch + 1], W[:, :, ch:ch + 1], d, ks,
                                     stride, nempty, grad=g[:, ch:ch + 1])
      assert np.allclose(out[:, ch:ch + 1], o1, atol=1e-12)
      assert np.allclose(gx[:, ch:ch + 1], gx1, atol=1e-12)
      assert np.allclose(gW[:, :, ch:ch + 1], gW1, atol=1e-12)


def test_tiny_pure_python(oct):
  # element-by-element loops, no vectorisation, on the first rows of a table
  d = 4
  table = oct.get_neigh(d, '333', 1, True)[:6]
  rows_in = int(oct.nnum_nempty[d])
  rng = np.random.default_rng(11)
  data = rng.standard_normal((rows_in, 2))
  W = rng.standard_normal((27, 2, 3))
  g = rng.standard_normal((6, 3))
  out = [[0.0] * 3 for _ in range(6)]
  gin = [[0.0] * 2 for _ in range(rows_in)]
  gw = [[[0.0] * 3 for _ in range(2)] for _ in range(27)]
  for i in range(6):
    for k in range(27):
      j = int(table[i, k])
      if j < 0:
        continue
      for a in range(2):
        for b in range(3):
          out[i][b] += data[j, a] * W[k, a, b]
          gin[j][a] += g[i, b] * W[k, a, b]
          gw[k][a][b] += data[j, a] * g[i, b]
  assert np.allclose(C.forward_gemm(data, W, table), np.array(out), atol=1e-12)
  assert np.allclose(C.backward_gemm(g, W, table, rows_in), np.array(gin), atol=1e-12)
  assert np.allclose(C.weight_gemm(data, g, table), np.array(gw), atol=1e-12)


def test_block_gemm_cpu_matches_definition(oct):
  # chunked torch form == definition; small max_buffer forces several chunks
  d, ci, co = 5, 4, 6
  table = oct.get_neigh(d, '333', 1, False)
  rows = table.shape[0]
  rng = np.random.default_rng(12)
  data = rng.standard_normal((rows, ci))
  W = rng.standard_normal((27, ci, co))
  g = rng.standard_normal((rows, co))
  eng = C.BlockGemmCPU(table, ci, max_buffer=int(2e4))
  assert eng.buffer_n > 1
  td, tW, tg = torch.from_numpy(data), torch.from_numpy(W), torch.from_numpy(g)
  assert np.allclose(eng.forward(td, tW).numpy(), C.forward_gemm(data, W, table), atol=1e-10)
  assert np.allclose(eng.backward(tg, tW, rows).numpy(),
                     C.backward_gemm(g, W, table, rows), atol=1e-10)
  assert np.allclose(eng.weight(td, tg, W.shape).numpy(),
                     C.weight_gemm(data, g, table), atol=1e-10)


def test_shape_check(oct):
  with pytest.raises(AssertionError):
    C.conv_layer(oct, np.zeros((3, 2)), np.zeros((27, 2, 2)), 4)


@pytest.mark.parametrize('kernel,stride,nempty', GRID)
def test_im2col_form_equals_the_engine(oct, kernel, stride, nempty):
  """octree2col + one matrix product is the forward pass, the product + col2octree the
  backward one (what the reference's explicit_gemm route computes, octree_conv.py:366-376,
  453-457), and col2octree is the adjoint of octree2col."""
  rng = np.random.default_rng(3)
  table = oct.get_neigh(5, kernel, stride, nempty)
  rows_in = int(oct.nnum_nempty[5] if nempty else oct.nnum[5])
  K = table.shape[1]
  data = rng.standard_normal((rows_in, 3))
  W = rng.standard_normal((K, 3, 4))
  col = C.octree2col(data, table)
  assert col.shape == (table.shape[0], K, 3)
  assert np.all(col[table < 0] == 0)
  np.testing.assert_allclose(col.reshape(len(table), -1) @ W.reshape(-1, 4), C.forward_gemm(data, W, table),
                             atol=1e-12)
  grad = rng.standard_normal((table.shape[0], 4))
  gcol = (grad @ W.reshape(-1, 4).T).reshape(len(table), K, 3)
  np.testing.assert_allclose(C.col2octree(gcol, table, rows_in), C.backward_gemm(grad, W, table, rows_in),
                             atol=1e-12)
  other = rng.standard_normal(col.shape)
  assert abs((col * other).sum() - (data * C.col2octree(other, table, rows_in)).sum()) < 1e-9
