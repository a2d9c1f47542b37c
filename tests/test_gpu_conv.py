"""GPU parity of OctreeConv / OctreeDeconv / OctreeDWConv (forward, data
gradient, weight gradient) through the C ABI against the fp64 oracle.

Tolerances (relative to the largest magnitude of the expected tensor):
  float32            1e-4
  float16, bfloat16  2e-2 against the fp64 result on the same (rounded) inputs
"""

import ctypes
import os
import sys

import numpy as np
import pytest
from conftest import random_cases
import torch

import ocnn_amd
from ocnn_amd import _lib, synthetic
from ocnn_amd.nn import (OctreeConv, OctreeConvTriton, OctreeDeconv, OctreeDWConv, octree_conv,
                         octree_conv_triton, octree_depad, octree_pad)
from ocnn_amd.octree import Octree, Points, merge_points
from oracle import conv_ref as C
from oracle import octree_ref as R

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def rel_err(got, want):
  got = got.detach().double().cpu().numpy()
  scale = max(1e-30, float(np.abs(want).max()))
  return float(np.abs(got - want).max()) / scale


def f64(t):
  return t.detach().double().cpu().numpy()


class Pair:
  """The same octree on the GPU (HIP path) and in the oracle."""

  def __init__(self, pts, nrm, bid, depth, full_depth, batch):
    pc = Points(pts.to(DEV), nrm.to(DEV), batch_id=None if bid is None else bid.to(DEV),
                batch_size=batch)
    self.gpu = Octree(depth, full_depth, batch_size=batch)
    self.gpu.build_octree(pc)
    self.gpu.construct_all_neigh()
    self.ref, _ = R.build_octree(pts.numpy(), nrm.numpy(),
                                 batch_id=None if bid is None else bid.numpy(), depth=depth,
                                 full_depth=full_depth, batch_size=batch)
    R.construct_all_neigh(self.ref)


@pytest.fixture(scope='module')
def small(ref_data):
  d4 = np.load(os.path.join(ref_data, 'octree/test_004.npz'))
  d5 = np.load(os.path.join(ref_data, 'octree/test_005.npz'))
  pts = torch.from_numpy(np.concatenate([d4['points'], d5['points']]))
  nrm = torch.from_numpy(np.concatenate([d4['normals'], d5['normals']]))
  bid = torch.cat([torch.zeros(len(d4['points']), 1), torch.ones(len(d5['points']), 1)])
  return Pair(pts, nrm, bid, 6, 3, 2)


@pytest.fixture(scope='module')
def medium():
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 3, 11, n=40000)
  return Pair(pts, nrm, bid, 7, 2, 3)


def rows_of(oct_ref, depth, nempty):
  return int(oct_ref.nnum_nempty[depth] if nempty else oct_ref.nnum[depth])


def run_layer(kind, pair, depth, ks, stride, nempty, cin, cout, dtype, seed=0, use_bias=True):
  """Runs module forward + backward on the GPU and the oracle; returns errors."""
  g = torch.Generator().manual_seed(seed)
  ks = (list(ks) + [ks[-1]] * 3)[:3]
  K = ks[0] * ks[1] * ks[2]
  if kind == 'conv':
    mod = OctreeConv(cin, cout, ks, stride, nempty, use_bias=use_bias)
    layer = C.conv_layer
  elif kind == 'deconv':
    mod = OctreeDeconv(cin, cout, ks, stride, nempty, use_bias=use_bias)
    layer = C.deconv_layer
  else:
    mod = OctreeDWConv(cin, ks, stride, nempty, use_bias=use_bias)
    layer = C.dwconv_layer
  with torch.no_grad():
    mod.weights.copy_(torch.randn(mod.weights.shape, generator=g) / (K * cin) ** 0.5)
    if use_bias:
      mod.bias.copy_(torch.randn(mod.bias.shape, generator=g))
  mod = mod.to(DEV).to(dtype)
  data = torch.randn(rows_of(pair.ref, depth, nempty), cin, generator=g).to(dtype)
  x = data.to(DEV).requires_grad_()
  out = mod(x, pair.gpu, depth)
  gout = torch.randn(out.shape, generator=g).to(dtype)
  out.backward(gout.to(DEV))
  bias = f64(mod.bias) if use_bias else None
  want = layer(pair.ref, f64(data), f64(mod.weights), depth, ks, stride, nempty, bias=bias,
               grad=f64(gout))
  assert tuple(out.shape) == want[0].shape
  errs = {'out': rel_err(out, want[0]), 'gdata': rel_err(x.grad, want[1]),
          'gw': rel_err(mod.weights.grad, want[2])}
  if use_bias:
    errs['gb'] = rel_err(mod.bias.grad, want[3])
  assert out.dtype == dtype and x.grad.dtype == dtype and mod.weights.grad.dtype == dtype
  return errs


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_fp32_modules_on_16_bit_features(medium, dtype):
  """Mixed precision as torch.amp leaves it (ocnn/nn/octree_conv.py:232,270: `weights.to(data.dtype)`):
  modules with fp32 parameters on 16-bit features give the bits of the all-16-bit run on the rounded
  parameters, and parameter gradients in fp32; the batch norm with fp32 parameters and buffers
  likewise matches its 16-bit twin to the rounding of the parameters."""
  from ocnn_amd.nn import BatchNormRelu1d
  g = torch.Generator().manual_seed(5)
  for kind, ks, stride, ne, cin, cout in [('conv', [3], 1, False, 64, 64), ('conv', [3], 1, True, 96, 96),
                                          ('conv', [2], 2, False, 32, 64), ('deconv', [2], 2, True, 64, 32),
                                          ('dwconv', [3], 1, False, 64, 64), ('conv', [3], 2, True, 48, 16)]:
    say('fp32 module on', dtype, kind, ks, stride, ne, cin, cout)
    Mod = {'conv': OctreeConv, 'deconv': OctreeDeconv}.get(kind)
    mod = OctreeDWConv(cin, ks, stride, ne, use_bias=True) if Mod is None else Mod(cin, cout, ks, stride, ne, use_bias=True)
    with torch.no_grad():
      mod.weights.copy_((torch.randn(mod.weights.shape, generator=g) / 30).to(dtype).float())   # values the dtype holds
      mod.bias.copy_(torch.randn(mod.bias.shape, generator=g).to(dtype).float())
    mod = mod.to(DEV)
    depth = 6 if kind == 'deconv' else 7
    rows = rows_of(medium.ref, depth, ne)
    x = torch.randn(rows, cin, generator=g).to(dtype).to(DEV).requires_grad_()
    out = mod(x, medium.gpu, depth)
    gout = torch.randn(out.shape, generator=g).to(dtype).to(DEV)
    out.backward(gout)
    assert out.dtype == dtype and x.grad.dtype == dtype
    assert mod.weights.grad.dtype == torch.float32 and mod.bias.grad.dtype == torch.float32
    import copy
    twin = copy.deepcopy(mod).to(dtype)
    twin.weights.grad = twin.bias.grad = None
    x2 = x.detach().clone().requires_grad_()
    out2 = twin(x2, medium.gpu, depth)
    out2.backward(gout)
    assert torch.equal(out, out2) and torch.equal(x.grad, x2.grad)
    assert torch.equal(mod.weights.grad, twin.weights.grad.float()) and torch.equal(mod.bias.grad, twin.bias.grad.float())
  for rows, c, relu in [(5000, 64, True), (777, 96, False)]:
    say('fp32 batch norm on', dtype, rows, c)
    bn = BatchNormRelu1d(c, relu=relu).to(DEV)
    with torch.no_grad():
      bn.weight.copy_((torch.rand(c, generator=g) + 0.5).to(dtype).float())
      bn.bias.copy_(torch.randn(c, generator=g).to(dtype).float())
    import copy
    twin = copy.deepcopy(bn).to(dtype)
    x = (torch.randn(rows, c, generator=g) + 1.0).to(dtype).to(DEV).requires_grad_()
    x2 = x.detach().clone().requires_grad_()
    dy = torch.randn(rows, c, generator=g).to(dtype).to(DEV)
    y, y2 = bn(x), twin(x2)
    y.backward(dy)
    y2.backward(dy)
    assert y.dtype == dtype and bn.weight.grad.dtype == torch.float32 and bn.running_mean.dtype == torch.float32
    assert torch.equal(y, y2) and torch.equal(x.grad, x2.grad)
    assert torch.allclose(bn.weight.grad, twin.weight.grad.float(), rtol=1e-2, atol=1e-2 * float(bn.weight.grad.abs().max()))
    assert torch.allclose(bn.running_var, twin.running_var.float(), rtol=1e-2, atol=1e-2)


GRID = [(k, s, ne) for k in ['333', '222', '311', '131', '113', '331', '313', '133']
        for s in (1, 2) for ne in (False, True)]


@pytest.mark.parametrize('kind', ['conv', 'deconv', 'dwconv'])
def test_fp32_grid(small, kind):
  """Every kernel shape x stride x nempty, fp32 (plain kernels, odd channels)."""
  for kern, stride, ne in GRID:
    ks = [int(c) for c in kern]
    depth = 4 if kind == 'deconv' else 5
    say('fp32', kind, kern, 'stride', stride, 'nempty', ne)
    errs = run_layer(kind, small, depth, ks, stride, ne, 5, 7, torch.float32)
    assert max(errs.values()) < TOL[torch.float32], (kind, kern, stride, ne, errs)


MFMA_SHAPES = [(32, 32), (64, 64), (64, 128), (128, 64), (32, 48), (96, 16)]


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_mfma_conv_333(small, medium, dtype):
  """3x3x3 stride-1 conv on the MFMA kernels, several channel shapes, both nempty modes."""
  for cin, cout in MFMA_SHAPES:
    for pair, depth in ((small, 6), (medium, 7), (medium, 5)):
      for ne in (False, True):
        say('mfma conv', dtype, cin, cout, 'depth', depth, 'nempty', ne)
        errs = run_layer('conv', pair, depth, [3], 1, ne, cin, cout, dtype)
        assert max(errs.values()) < TOL[dtype], (cin, cout, depth, ne, errs)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_mfma_stride2_deconv_dw(medium, dtype):
  """The child/parent paths: 2x2x2 stride-2 conv and deconv, 3x3x3 stride-2,
  and the depth-wise kernel, in 16-bit types."""
  for ne in (False, True):
    say('mfma s2 conv 64->128', dtype, ne)
    errs = run_layer('conv', medium, 7, [2], 2, ne, 64, 128, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    say('mfma s2 deconv 128->64', dtype, ne)
    errs = run_layer('deconv', medium, 6, [2], 2, ne, 128, 64, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    say('mfma s2 conv 333 32->32', dtype, ne)
    errs = run_layer('conv', medium, 7, [3], 2, ne, 32, 32, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    say('mfma s1 deconv 333 32->64', dtype, ne)
    errs = run_layer('deconv', medium, 6, [3], 1, ne, 32, 64, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    say('dwconv 128', dtype, ne)
    errs = run_layer('dwconv', medium, 6, [3], 1, ne, 128, 128, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    errs = run_layer('dwconv', medium, 7, [2], 2, ne, 24, 24, dtype)
    assert max(errs.values()) < TOL[dtype], errs
    # more channels than a workgroup has threads (every channel's weight gradient must be written)
    say('dwconv s2 512', dtype, ne)
    errs = run_layer('dwconv', medium, 6, [2], 2, ne, 512, 512, dtype)
    assert max(errs.values()) < TOL[dtype], errs


def test_fp32_larger(medium):
  say('fp32 32->32 at depth 6 (the CPU-runnable reference case shape)')
  errs = run_layer('conv', medium, 6, [3], 1, False, 32, 32, torch.float32)
  assert max(errs.values()) < TOL[torch.float32], errs
  errs = run_layer('conv', medium, 6, [3], 1, True, 32, 32, torch.float32)
  assert max(errs.values()) < TOL[torch.float32], errs
  # fp32 on the MFMA kernels as bf16 pieces: every layer kind and table form, still 1e-4
  for kind, depth, ks, stride, ne, cin, cout in [
      ('conv', 7, [3], 1, False, 64, 64), ('conv', 7, [2], 2, False, 64, 128),
      ('conv', 7, [2], 2, True, 32, 64), ('deconv', 6, [2], 2, False, 128, 64),
      ('deconv', 6, [3], 1, True, 32, 32), ('conv', 6, [3], 2, False, 32, 48),
      ('conv', 6, [3, 1, 3], 1, False, 64, 32)]:
    say('fp32 via bf16 pieces', kind, depth, ks, stride, ne, cin, cout)
    errs = run_layer(kind, medium, depth, ks, stride, ne, cin, cout, torch.float32)
    assert max(errs.values()) < TOL[torch.float32], (kind, ks, stride, ne, cin, cout, errs)


def test_mixed_precision_and_no_bias(small):
  say('fp32 parameters with fp16 data (weights cast inside, grads cast back)')
  conv = OctreeConv(32, 32, [3], 1, nempty=True, use_bias=False).to(DEV)
  data = torch.randn(rows_of(small.ref, 6, True), 32, generator=torch.Generator().manual_seed(1))
  x = data.half().to(DEV).requires_grad_()
  out = conv(x, small.gpu, 6)
  assert out.dtype == torch.float16
  out.sum().backward()
  assert conv.weights.grad.dtype == torch.float32 and x.grad.dtype == torch.float16
  want = C.conv_layer(small.ref, f64(data.half()), f64(conv.weights.half()), 6, [3], 1, True)
  assert rel_err(out, want) < 2e-2


def test_table_level_api(small):
  say('octree_conv_triton(data, weight(Co,V,Ci), bias, neigh) parity with the module')
  g = torch.Generator().manual_seed(5)
  cin, cout, depth = 32, 64, 6
  neigh = small.gpu.get_neigh(depth, '333', 1, False)            # int64, as the reference passes
  w = (torch.randn(27, cin, cout, generator=g) / 30).half().to(DEV).requires_grad_()
  b = torch.randn(cout, generator=g).half().to(DEV).requires_grad_()
  x = torch.randn(neigh.shape[0], cin, generator=g).half().to(DEV).requires_grad_()
  out = octree_conv_triton(x, w.permute(2, 0, 1), b, neigh)
  gout = torch.randn(out.shape, generator=g).half().to(DEV)
  out.backward(gout)
  want = C.conv_layer(small.ref, f64(x), f64(w), depth, [3], 1, False, bias=f64(b), grad=f64(gout))
  assert rel_err(out, want[0]) < 2e-2 and rel_err(x.grad, want[1]) < 2e-2
  assert rel_err(w.grad, want[2]) < 2e-2 and rel_err(b.grad, want[3]) < 2e-2
  mod = OctreeConvTriton(cin, cout, [3], 1, use_bias=True).to(DEV).half()
  with torch.no_grad():
    mod.weights.copy_(w)
    mod.bias.copy_(b)
  assert rel_err(mod(x.detach(), small.gpu, depth), want[0]) < 2e-2


@pytest.mark.parametrize('nempty', [False, True])
def test_octree2col_and_col2octree(small, nempty):
  say('octree2col / col2octree against the oracle, all kernel shapes and strides, nempty', nempty)
  from ocnn_amd.nn import col2octree, octree2col
  g = torch.Generator().manual_seed(12)
  d = 5
  rows_in = rows_of(small.ref, d, nempty)
  data = torch.randn(rows_in, 5, generator=g)
  for kern in ['333', '222', '311', '131', '113', '331', '313', '133']:
    for stride in (1, 2):
      table = small.ref.get_neigh(d, kern, stride, nempty)
      col = octree2col(data.to(DEV), small.gpu, d, kern, stride, nempty)
      want = C.octree2col(f64(data), table)
      assert col.dtype == torch.float32 and np.array_equal(f64(col), want), (kern, stride)
      other = torch.randn(col.shape, generator=g)
      back = col2octree(other.to(DEV), small.gpu, d, kern, stride, nempty)
      assert rel_err(back, C.col2octree(f64(other), table, rows_in)) < 1e-6, (kern, stride)


@pytest.mark.parametrize('kind', ['conv', 'deconv'])
def test_explicit_gemm_equals_the_hip_engine(small, kind):
  """The reference's own cross-check (test/test_octree_conv.py:85-163): the im2col route
  through autograd against the engine, output, data gradient and weight gradient, over kernel
  shapes x strides x nempty, fp32."""
  g = torch.Generator().manual_seed(13)
  depth, cin, cout = 5, 6, 7
  Mod = OctreeConv if kind == 'conv' else OctreeDeconv
  for kern, stride, ne in GRID:
    ks = [int(c) for c in kern]
    mods = [Mod(cin, cout, ks, stride, ne, method=m, use_bias=True).to(DEV) for m in ('explicit_gemm', 'hip')]
    assert mods[0].method == 'explicit_gemm' and mods[1].method == 'hip'
    with torch.no_grad():
      mods[0].bias.copy_(torch.randn(cout, generator=g))
      mods[1].weights.copy_(mods[0].weights)
      mods[1].bias.copy_(mods[0].bias)
    data = torch.randn(rows_of(small.ref, depth, ne), cin, generator=g)
    res = []
    for m in mods:
      x = data.to(DEV).requires_grad_()
      out = m(x, small.gpu, depth)
      if not res:
        gout = torch.randn(out.shape, generator=g).to(DEV)
      out.backward(gout)
      res.append((out, x.grad, m.weights.grad, m.bias.grad))
    for name, a, b in zip(('out', 'gdata', 'gw', 'gb'), res[0], res[1]):
      assert a.shape == b.shape, (kind, kern, stride, ne, name)
      assert rel_err(b, f64(a)) < 1e-4, (kind, kern, stride, ne, name)


def test_pad_depad(small):
  say('octree_pad / octree_depad')
  d = 5
  x = torch.randn(int(small.ref.nnum_nempty[d]), 6).to(DEV).requires_grad_()
  p = octree_pad(x, small.gpu, d, val=1.5)
  assert np.array_equal(f64(p), C.octree_pad(f64(x), small.ref, d, 1.5))
  assert torch.equal(octree_depad(p, small.gpu, d), x.detach())
  p.sum().backward()
  assert torch.equal(x.grad, torch.ones_like(x))
  for dt in (torch.float16, torch.bfloat16):
    y = torch.randn(int(small.ref.nnum[d]), 9).to(dt).to(DEV)
    assert np.array_equal(f64(octree_depad(y, small.gpu, d)), C.octree_depad(f64(y), small.ref, d))


def test_errors(small):
  say('error behaviour')
  conv = OctreeConv(4, 4).to(DEV)
  with pytest.raises(AssertionError):
    conv(torch.zeros(3, 4, device=DEV), small.gpu, 5)
  with pytest.raises(RuntimeError):
    conv(torch.zeros(int(small.ref.nnum[5]), 4), small.gpu, 5)        # CPU tensor: no fallback
  with pytest.raises(TypeError):
    conv.double()(torch.zeros(int(small.ref.nnum[5]), 4, device=DEV, dtype=torch.double),
                  small.gpu, 5)
  with pytest.raises(ValueError):
    OctreeConv(4, 4, [5]).to(DEV)(torch.zeros(int(small.ref.nnum[5]), 4, device=DEV), small.gpu, 5)


def test_weight_gradient_is_bit_reproducible(medium):
  say('two runs of the split-K weight gradient give identical bits')
  g = torch.Generator().manual_seed(9)
  t = medium.gpu._table(7, '333', 1, False)
  x = torch.randn(t.shape[0], 64, generator=g).bfloat16().to(DEV)
  gr = torch.randn(t.shape[0], 64, generator=g).bfloat16().to(DEV)
  a = ocnn_amd.nn.conv_wgrad(x, gr, t)
  b = ocnn_amd.nn.conv_wgrad(x, gr, t)
  assert torch.equal(a, b)


def test_benchmark_shape_properties():
  """Depth 8, batch 8, 64->64, fp16 and bf16 at the benchmark size: adjoint and
  bilinear identities (size independent), plus a sampled oracle comparison."""
  say('benchmark-size properties: build')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 8, 1001, n=100000)
  pc = Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=8)
  o = Octree(8, 2, batch_size=8)
  o.build_octree(pc)
  o.construct_all_neigh()
  rows = int(o.nnum[8])
  g = torch.Generator().manual_seed(2)
  for dtype in (torch.float16, torch.bfloat16):
    say('benchmark-size properties:', dtype, rows, 'rows')
    conv = OctreeConv(64, 64, [3], 1).to(DEV).to(dtype)
    x = torch.randn(rows, 64, generator=g).to(dtype).to(DEV).requires_grad_()
    out = conv(x, o, 8)
    gout = torch.randn(rows, 64, generator=g).to(dtype).to(DEV)
    out.backward(gout)
    lhs = (out.double() * gout.double()).sum().item()
    rhs_x = (x.detach().double() * x.grad.double()).sum().item()
    rhs_w = (conv.weights.detach().double() * conv.weights.grad.double()).sum().item()
    scale = (out.double().norm() * gout.double().norm()).item()
    assert abs(lhs - rhs_x) / scale < 2e-3, (lhs, rhs_x, scale)
    assert abs(lhs - rhs_w) / scale < 2e-3, (lhs, rhs_w, scale)
    # sampled rows against the definition, from the GPU table itself
    t = o._table(8, '333', 1, False)
    sel = torch.randint(0, rows, (512,), generator=g)
    tt = t[sel.to(DEV)].cpu().numpy()
    xd, wd = f64(x), f64(conv.weights)
    want = np.zeros((512, 64))
    for k in range(27):
      v = tt[:, k] >= 0
      want[v] += xd[tt[v, k]] @ wd[k]
    assert rel_err(out[sel.to(DEV)], want) < TOL[dtype]


def test_tile_plan_reconstructs_table(medium):
  say('tile plan: distinct-row lists and positions reproduce the table')
  from ocnn_amd.octree.octree import TilePlan
  for kern, stride, ne in [('333', 1, False), ('333', 1, True), ('222', 2, False)]:
    t = medium.gpu._table(7, kern, stride, ne)
    plan = TilePlan(t)
    tab = t.cpu().numpy()
    loc = plan.loc.cpu().numpy().view(np.uint16)
    uptr = plan.uptr.cpu().numpy()
    urows = plan.urows.cpu().numpy()
    R = _lib.lib().ocnn_tile_plan_rows()
    assert uptr[0] == 0 and uptr[-1] == plan.total
    for tile in range(0, (tab.shape[0] + R - 1) // R, 7):
      blk = tab[tile * R:(tile + 1) * R]
      u = urows[uptr[tile]:uptr[tile + 1]]
      assert np.array_equal(u, np.unique(blk[blk >= 0])), tile
      lb = loc[tile].T[:blk.shape[0]]                      # (slot, row) -> (row, slot)
      assert (loc[tile].T[blk.shape[0]:] == 0).all()       # rows past the table: empty
      assert np.array_equal(lb == 0, blk < 0)              # 0 = empty, else position + 1
      assert np.array_equal(u[lb[blk >= 0] - 1], blk[blk >= 0])


def test_tile_plan_of_tables_without_locality():
  """Tiles whose entries name thousands of scattered rows do not fit the small set of the
  one-pass build: the plan is then built the long way and still reproduces the table, whether
  all tiles are like that or a few among local ones (those few are dropped from the plan and
  listed as overflow rows)."""
  from ocnn_amd.octree.octree import TilePlan
  R = _lib.lib().ocnn_tile_plan_rows()
  g = torch.Generator().manual_seed(17)
  rows, K = 40 * R + 37, 27
  scattered = torch.randint(0, 1 << 20, (rows, K), generator=g, dtype=torch.int32)
  scattered[torch.rand(rows, K, generator=g) < 0.2] = -1
  local = (torch.arange(rows, dtype=torch.int32).view(-1, 1) + torch.randint(-60, 60, (rows, K), generator=g,
                                                                              dtype=torch.int32)).clamp_(0, rows - 1)
  mixed = local.clone()
  mixed[3 * R:4 * R] = scattered[3 * R:4 * R]
  mixed[17 * R:18 * R] = scattered[17 * R:18 * R]
  for name, t in (('scattered', scattered), ('mixed', mixed), ('local', local)):
    say('tile plan without locality:', name)
    plan = TilePlan(t.to(DEV))
    tab = t.numpy().copy()
    if name == 'mixed':
      want = np.concatenate([np.arange(3 * R, 4 * R), np.arange(17 * R, 18 * R)])
      assert np.array_equal(plan.overflow_rows.cpu().numpy(), want)
      assert np.array_equal(plan.overflow_table.cpu().numpy(), tab[want])
      tab[want] = -1                                         # those tiles are empty in the plan
    else:
      assert plan.overflow_rows is None
    assert (plan.umax > TilePlan.CAP) == (name == 'scattered')
    loc = plan.loc.cpu().numpy().view(np.uint16)
    uptr = plan.uptr.cpu().numpy()
    urows = plan.urows.cpu().numpy()
    assert uptr[0] == 0 and uptr[-1] == plan.total
    for tile in range((rows + R - 1) // R):
      blk = tab[tile * R:(tile + 1) * R]
      u = urows[uptr[tile]:uptr[tile + 1]]
      assert np.array_equal(u, np.unique(blk[blk >= 0])), (name, tile)
      lb = loc[tile].T[:blk.shape[0]]
      assert np.array_equal(lb == 0, blk < 0)
      assert np.array_equal(u[lb[blk >= 0] - 1], blk[blk >= 0])


def _same_plan(a, b):
  assert (a.rows, a.K, a.total, a.umax, a.nnz) == (b.rows, b.K, b.total, b.umax, b.nnz)
  assert torch.equal(a.uptr, b.uptr) and torch.equal(a.urows[:a.total], b.urows[:b.total]) and torch.equal(a.loc, b.loc)
  assert (a.overflow_rows is None) == (b.overflow_rows is None)
  if a.overflow_rows is not None:
    assert torch.equal(a.overflow_rows, b.overflow_rows) and torch.equal(a.overflow_table, b.overflow_table)


def _same_pairs(a, b):
  assert (a.n_lists, a.n_blocks, a.max_blocks) == (b.n_lists, b.n_blocks, b.max_blocks)
  assert list(a.lists_host) == list(b.lists_host) and list(a.list_count_host) == list(b.list_count_host)
  assert list(a.group_bounds_host) == list(b.group_bounds_host)
  assert torch.equal(a.lists, b.lists) and torch.equal(a.cptr, b.cptr)
  assert torch.equal(a.ent[:16 * a.n_blocks], b.ent[:16 * b.n_blocks])


def test_plans_built_together_equal_plans_built_alone(medium):
  say('tile plans and pair plans: one read-back for several tables gives the same plans')
  from ocnn_amd.octree.octree import PairPlan, TilePlan
  o = medium.gpu
  tables = [o._table(7, '333', 1, False), o._table(7, '333', 1, True), o._table(7, '222', 2, True),
            o._table_t(7, '222', 2, True, int(o.nnum_nempty[7])), o._table(6, '313', 1, True),
            torch.empty((0, 27), dtype=torch.int32, device=DEV)]
  alone = [TilePlan(t) for t in tables]
  together = TilePlan.build_many(tables)
  for a, b in zip(alone, together):
    _same_plan(a, b)
  # a low staging limit: some tiles overflow (emptied in the plan), and one table has too many
  counts = (alone[1].uptr[1:] - alone[1].uptr[:-1]).float()
  cap = int(torch.quantile(counts, 0.97))
  alone = [TilePlan(t, cap=cap) for t in tables]
  together = TilePlan.build_many(tables, cap=cap)
  assert any(p.overflow_rows is not None for p in alone)
  for a, b in zip(alone, together):
    _same_plan(a, b)
  for a, b in zip([PairPlan(p) for p in alone], PairPlan.build_many(together)):
    _same_pairs(a, b)


def test_fresh_octree_builds_the_plans_of_its_predecessors(medium):
  say('plans: a fresh octree builds what earlier octrees were asked for, at its first request')
  def fresh():
    o = Octree(7, 2, batch_size=3)
    pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 3, 11, n=40000)
    o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=3))
    o.construct_all_neigh()
    return o
  from ocnn_amd.octree.octree import PlanHistory
  saved = Octree.plan_history
  Octree.plan_history = PlanHistory()
  try:
    first = fresh()
    keys = [(7, '333', 1, True, False), (6, '333', 1, True, False), (7, '222', 2, True, False),
            (7, '222', 2, True, True), (5, '333', 1, False, False)]
    for d, k, s, ne, inv in keys:
      p = first._plan(d, k, s, ne, inv, first._fine_rows(d, ne))
      if d == 7 and k == '333':
        p.pairs()
    assert len(first._plans) == len(keys)
    second = fresh()
    assert not second._plans
    second._plan(5, '333', 1, False, False, None)            # any request builds all of them
    assert set(second._plans) == set(first._plans)
    for ck, p in first._plans.items():
      _same_plan(p, second._plans[ck])
      assert (p._pairs is None) == (second._plans[ck]._pairs is None)
      if p._pairs is not None:
        _same_pairs(p._pairs, second._plans[ck]._pairs)
    # switched off: plans are built one by one, on request
    Octree.PREBUILD_PLANS = False
    third = fresh()
    third._plan(5, '333', 1, False, False, None)
    assert len(third._plans) == 1
  finally:
    Octree.PREBUILD_PLANS = True
    Octree.plan_history = saved


def test_octree_prepared_on_a_side_stream():
  say('plans: an octree built and prepared on a second stream while the first one works')
  def fresh():
    o = Octree(7, 2, batch_size=3)
    pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 3, 11, n=40000)
    o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=3))
    o.construct_all_neigh()
    return o
  from ocnn_amd.octree.octree import PlanHistory
  saved = Octree.plan_history
  Octree.plan_history = PlanHistory()
  try:
    torch.manual_seed(3)
    layers = [ocnn_amd.nn.OctreeConv(64, 64, [3], 1, nempty=True).to(DEV).bfloat16(),
              ocnn_amd.nn.OctreeConv(64, 96, [2], 2, nempty=True).to(DEV).bfloat16(),
              ocnn_amd.nn.OctreeDeconv(96, 64, [2], 2, nempty=True).to(DEV).bfloat16()]
    def run(o, x):
      x = x.clone().requires_grad_()
      y = layers[0](x, o, 7)
      z = layers[2](layers[1](y, o, 7), o, 6)
      for l in layers:
        l.weights.grad = None
      (y + z).float().square().sum().backward()
      return [z.detach().clone(), x.grad.clone()] + [l.weights.grad.clone() for l in layers]
    first = fresh()
    assert first.prepare() is first and not first._plans          # nothing asked for yet: nothing built
    x = torch.randn(int(first.nnum_nempty[7]), 64, device=DEV).bfloat16()
    want = run(first, x)
    assert first.prepare() is first and len(first._plans) >= 3      # (nothing left to build)
    side, main = torch.cuda.Stream(), torch.cuda.current_stream()
    torch.cuda.synchronize()
    for rep in range(3):
      # main gets a queue of work; the next octree is built beside it
      for _ in range(4):
        run(first, x)
      with torch.cuda.stream(side):
        nxt = fresh().prepare()
      assert set(nxt._plans) == set(first._plans)
      main.wait_stream(side)
      nxt.record_stream(main)
      got = run(nxt, x)
      del nxt
      for a, b in zip(want, got):
        assert torch.equal(a, b), rep
  finally:
    Octree.plan_history = saved


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_staged_kernel_many_passes(dtype):
  """A table with no locality: tiles need far more distinct rows than fit in
  LDS at once, so the staged kernel takes several passes per tile."""
  say('staged gather-GEMM on a random table (multi-pass)', dtype)
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(21)
  rows_in, rows, K, cin, cout = 6000, 300, 27, 128, 64
  table = torch.randint(0, rows_in, (rows, K), generator=g, dtype=torch.int32)
  table[torch.rand(rows, K, generator=g) < 0.3] = -1
  x = torch.randn(rows_in, cin, generator=g).to(dtype)
  w = (torch.randn(K, cin, cout, generator=g) / 40).to(dtype)
  b = torch.randn(cout, generator=g).to(dtype)
  tg = table.to(DEV)
  plan = TilePlan(tg)
  assert int((plan.uptr[1:] - plan.uptr[:-1]).max()) > 320
  plan.reuse = 10.0          # a random table has no reuse; make the layer above take the staged kernel anyway
  got = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), cout, False, False, b.to(DEV), plan)
  want = C.forward_gemm(f64(x), f64(w), table.numpy().astype(np.int64)) + f64(b)
  assert rel_err(got, want) < TOL[dtype]
  old = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), cout, False, False, b.to(DEV))
  assert rel_err(old, want) < TOL[dtype]
  # transposed + mirrored weights through the same plan
  wt = (torch.randn(K, cout, cin, generator=g) / 40).to(dtype)
  got = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, wt.to(DEV), cout, True, True, None, plan)
  want = C.forward_gemm(f64(x), np.ascontiguousarray(f64(wt)[::-1].transpose(0, 2, 1)),
                        table.numpy().astype(np.int64))
  assert rel_err(got, want) < TOL[dtype]


def _local_table(rows, rows_in, K, g, spread=40, empty=0.3):
  """A table with the locality of an octree neighbourhood: entry (r, k) points near
  r * rows_in / rows, so a 128-row tile touches a few hundred distinct rows."""
  base = (torch.arange(rows, dtype=torch.float64) * (rows_in / max(rows, 1))).long()[:, None]
  off = torch.randint(-spread, spread + 1, (rows, K), generator=g)
  t = (base + off).clamp_(0, rows_in - 1).to(torch.int32)
  t[torch.rand(rows, K, generator=g) < empty] = -1
  return t


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K', [27, 9, 8, 3])
@pytest.mark.parametrize('ch', [64, 32])
def test_planned_64x64_kernels(dtype, K, ch):
  """The persistent 64 -> 64 and 32 -> 32 kernels (gather-GEMM with register-resident weights,
  weight gradient on the tile plan) for every slot count they are built for, on
  tables whose row count is not a multiple of the tile, against the oracle and
  against the plan-free kernels."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(100 + K)
  for rows, rows_in in [(1000, 1000), (4133, 2300), (130, 150), (128 * 300 + 1, 128 * 300 + 1)]:
    say('planned kernels', dtype, 'K', K, 'rows', rows, 'rows_in', rows_in)
    table = _local_table(rows, rows_in, K, g)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
    assert L.ocnn_conv_gather_rw_supported(code, rows_in, K, ch, ch, plan.umax)
    assert L.ocnn_conv_wgrad_planned_supported(code, rows_in, rows, K, ch, ch, plan.umax)
    x = torch.randn(rows_in, ch, generator=g).to(dtype)
    w = (torch.randn(K, ch, ch, generator=g) / (K * ch) ** 0.5).to(dtype)
    b = torch.randn(ch, generator=g).to(dtype)
    gr = torch.randn(rows, ch, generator=g).to(dtype)
    t64 = table.numpy().astype(np.int64)
    # gather-GEMM, with bias
    got = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), ch, False, False, b.to(DEV), plan)
    want = C.forward_gemm(f64(x), f64(w), t64) + f64(b)
    assert rel_err(got, want) < TOL[dtype]
    # transposed, mirrored weights (the data gradient of a symmetric table)
    got = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), ch, True, True, None, plan)
    want = C.forward_gemm(f64(x), np.ascontiguousarray(f64(w)[::-1].transpose(0, 2, 1)), t64)
    assert rel_err(got, want) < TOL[dtype]
    # weight gradient, both output layouts; same bits on a second run
    gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
    want = C.weight_gemm(f64(x), f64(gr), t64)
    assert rel_err(gw, want) < TOL[dtype]
    assert rel_err(ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg), want) < TOL[dtype]
    gwt = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, True, plan)
    assert torch.equal(gwt, gw.transpose(1, 2).contiguous())
    assert torch.equal(gw, ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan))


@pytest.mark.parametrize('K,ca,cb', [(27, 32, 32), (27, 64, 64), (9, 64, 128), (8, 128, 64), (3, 32, 32), (27, 96, 160)])
def test_planned_weight_gradient_fp32(K, ca, cb):
  """fp32 tensors on the planned weight-gradient kernel (two bf16 pieces per value, three passes,
  one reduction): 1e-4 of the fp64 sums, the same bits on a second run, both output layouts,
  and the selection takes it."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(200 + K + ca)
  for rows, rows_in in [(1000, 1000), (4133, 2300), (128 * 300 + 1, 128 * 300 + 1)]:
    say('planned weight gradient, fp32', 'K', K, ca, cb, 'rows', rows, 'rows_in', rows_in)
    table = _local_table(rows, rows_in, K, g)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    assert L.ocnn_conv_wgrad_planned_supported(0, rows_in, rows, K, ca, cb, plan.umax)
    assert L.ocnn_conv_wgrad_choose(0, rows_in, rows, K, ca, cb, 0, 1, plan.umax, plan.total,
                                    float(plan.occupancy)) == _lib.WGRAD_PLANNED
    x = torch.randn(rows_in, ca, generator=g)
    gr = torch.randn(rows, cb, generator=g)
    want = C.weight_gemm(f64(x), f64(gr), table.numpy().astype(np.int64))
    gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
    assert gw.dtype == torch.float32 and rel_err(gw, want) < 1e-4, rel_err(gw, want)
    assert torch.equal(gw, ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan))
    gwt = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, True, plan)
    assert torch.equal(gwt, gw.transpose(1, 2).contiguous())


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('cin,cout', [(64, 128), (128, 512), (512, 128), (256, 256), (1024, 384), (192, 1024)])
def test_dense_rows_kernel(dtype, cin, cout):
  """out = in W + bias on the kernel for one-slot identity tables (every row-block and
  output-channel tiling it is built with), both weight layouts, ragged row counts."""
  L = _lib.lib()
  g = torch.Generator().manual_seed(cin + cout)
  code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
  for rows in (1, 130, 4133):
    say('dense rows', dtype, cin, cout, rows)
    assert L.ocnn_conv_dense_supported(code, rows, cin, cout)
    x = torch.randn(rows, cin, generator=g).to(dtype)
    w = (torch.randn(cin, cout, generator=g) / cin ** 0.5).to(dtype)
    b = torch.randn(cout, generator=g).to(dtype)
    want = f64(x) @ f64(w) + f64(b)
    for transposed in (0, 1):
      wd = (w.t().contiguous() if transposed else w).to(DEV)
      out = torch.empty((rows, cout), dtype=dtype, device=DEV)
      ws = torch.empty(cin * cout * 2, dtype=torch.uint8, device=DEV)
      xd, bd = x.to(DEV), b.to(DEV)
      _lib.check(L.ocnn_conv_dense(code, _lib.ptr(xd), rows, _lib.ptr(wd), cin, cout, transposed, _lib.ptr(bd),
                                   _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
      assert rel_err(out, want) < TOL[dtype]


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('cin,cout', [(128, 512), (512, 128), (64, 128), (256, 256), (96, 64)])
def test_dense_rows_register_kernels_indexed(dtype, cin, cout):
  """The same kernels with the rows of an operand taken through an index (the rows of the
  non-empty nodes read out of a tensor over all nodes): bit-identical to the kernels run on the
  rows copied out first, for ragged row counts, fewer tiles than the rings hold, an index that
  is the identity and one with gaps, and guard rows around the output."""
  L = _lib.lib()
  g = torch.Generator().manual_seed(5 * cin + cout)
  code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
  for rows, total in ((1, 9), (130, 130), (4133, 9000), (64 * 300 + 5, 64 * 800)):
    say('dense rows rw indexed', dtype, cin, cout, rows, total)
    index = torch.sort(torch.randperm(total, generator=g)[:rows]).values.to(torch.int32)
    x_all = torch.randn(total, cin, generator=g).to(dtype).to(DEV)
    g_all = torch.randn(total, cout, generator=g).to(dtype).to(DEV)
    x_own = torch.randn(rows, cin, generator=g).to(dtype).to(DEV)
    idx = index.to(DEV)
    x_sel, g_sel = x_all.index_select(0, idx.long()), g_all.index_select(0, idx.long())
    if L.ocnn_conv_dense_rw_supported(code, rows, cin, cout):
      w = (torch.randn(cin, cout, generator=g) / cin ** 0.5).to(dtype).to(DEV)
      b = torch.randn(cout, generator=g).to(dtype).to(DEV)
      ws = torch.empty(cin * cout * 2, dtype=torch.uint8, device=DEV)
      want = torch.empty((rows, cout), dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_rw(code, _lib.ptr(x_sel), rows, _lib.ptr(w), cin, cout, 0, _lib.ptr(b),
                                      _lib.ptr(want), _lib.ptr(ws), ws.numel(), _lib.stream()))
      out = torch.full((rows + 1, cout), 7.0, dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_rw_indexed(code, _lib.ptr(x_all), total, _lib.ptr(idx), rows, _lib.ptr(w), cin,
                                              cout, 0, _lib.ptr(b), _lib.ptr(out), rows, None, _lib.ptr(ws),
                                              ws.numel(), _lib.stream()))
      assert torch.equal(out[:rows], want) and bool((out[rows] == 7.0).all())
      assert rel_err(out[:rows], f64(x_sel) @ f64(w) + f64(b)) < TOL[dtype]
      # the result through the index too: its rows land at the index's rows of a larger tensor,
      # the other rows are not touched; ocnn_pad without data then zeroes the rows of the gaps
      spread = torch.full((total, cout), 7.0, dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_rw_indexed(code, _lib.ptr(x_all), total, _lib.ptr(idx), rows, _lib.ptr(w), cin,
                                              cout, 0, _lib.ptr(b), _lib.ptr(spread), total, _lib.ptr(idx),
                                              _lib.ptr(ws), ws.numel(), _lib.stream()))
      assert torch.equal(spread.index_select(0, idx.long()), want)
      gaps = torch.ones(total, dtype=torch.bool, device=DEV)
      gaps[idx.long()] = False
      assert bool((spread[gaps] == 7.0).all())
      children = torch.full((total,), -1, dtype=torch.int32, device=DEV)
      children[idx.long()] = torch.arange(rows, dtype=torch.int32, device=DEV)
      _lib.check(L.ocnn_pad(code, None, _lib.ptr(children), total, cout, 0.0, _lib.ptr(spread), _lib.stream()))
      assert torch.equal(spread.index_select(0, idx.long()), want) and not bool(spread[gaps].any())
    ws = torch.empty(L.ocnn_conv_dense_wgrad_rw_workspace_bytes(cin, cout), dtype=torch.uint8, device=DEV)
    want = torch.empty((cin, cout), dtype=dtype, device=DEV)
    _lib.check(L.ocnn_conv_dense_wgrad_rw(code, _lib.ptr(x_own), _lib.ptr(g_sel), rows, cin, cout, 0,
                                          _lib.ptr(want), _lib.ptr(ws), ws.numel(), _lib.stream()))
    gw = torch.empty((cin, cout), dtype=dtype, device=DEV)
    _lib.check(L.ocnn_conv_dense_wgrad_rw_indexed(code, _lib.ptr(x_own), rows, None, _lib.ptr(g_all), total,
                                                  _lib.ptr(idx), rows, cin, cout, 0, _lib.ptr(gw), _lib.ptr(ws),
                                                  ws.numel(), _lib.stream()))
    assert torch.equal(gw, want)
    assert rel_err(gw, f64(x_own).T @ f64(g_sel)) < TOL[dtype]
    # both operands through the index
    _lib.check(L.ocnn_conv_dense_wgrad_rw(code, _lib.ptr(x_sel), _lib.ptr(g_sel), rows, cin, cout, 0,
                                          _lib.ptr(want), _lib.ptr(ws), ws.numel(), _lib.stream()))
    _lib.check(L.ocnn_conv_dense_wgrad_rw_indexed(code, _lib.ptr(x_all), total, _lib.ptr(idx), _lib.ptr(g_all), total,
                                                  _lib.ptr(idx), rows, cin, cout, 0, _lib.ptr(gw), _lib.ptr(ws),
                                                  ws.numel(), _lib.stream()))
    assert torch.equal(gw, want)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('cin,cout', [(64, 128), (64, 512), (128, 128), (128, 256), (128, 512), (256, 128), (256, 256),
                                      (512, 128), (512, 384), (1024, 128), (128, 1024), (96, 64), (768, 96),
                                      (64, 16), (128, 96), (384, 256), (72, 40), (256, 32), (8, 8)])
def test_dense_rows_register_kernels(dtype, cin, cout):
  """The persistent kernels for one-slot identity tables: out = in W + bias with the weights
  in registers (every input width / output blocking they are built with, both weight layouts),
  and gw = x^T g with the sums in registers (every block shape, also channel counts that fill
  only a part of a block), ragged row counts, fewer tiles than the ring of buffers holds."""
  L = _lib.lib()
  g = torch.Generator().manual_seed(3 * cin + cout)
  code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
  for rows in (1, 130, 4133, 64 * 300):
    say('dense rows rw', dtype, cin, cout, rows)
    x = torch.randn(rows, cin, generator=g).to(dtype)
    gr = torch.randn(rows, cout, generator=g).to(dtype)
    xd, gd = x.to(DEV), gr.to(DEV)
    if L.ocnn_conv_dense_rw_supported(code, rows, cin, cout):
      w = (torch.randn(cin, cout, generator=g) / cin ** 0.5).to(dtype)
      b = torch.randn(cout, generator=g).to(dtype)
      want = f64(x) @ f64(w) + f64(b)
      for transposed in (0, 1):
        wd = (w.t().contiguous() if transposed else w).to(DEV)
        out = torch.full((rows + 1, cout), 7.0, dtype=dtype, device=DEV)      # one guard row
        ws = torch.empty(cin * cout * 2, dtype=torch.uint8, device=DEV)
        bd = b.to(DEV)
        _lib.check(L.ocnn_conv_dense_rw(code, _lib.ptr(xd), rows, _lib.ptr(wd), cin, cout, transposed,
                                        _lib.ptr(bd), _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
        assert rel_err(out[:rows], want) < TOL[dtype]
        assert bool((out[rows] == 7.0).all())
    else:
      assert cin not in (64, 128, 256, 512) or cout % 128
    assert L.ocnn_conv_dense_wgrad_rw_supported(code, rows, cin, cout)     # any multiples of 8
    if True:
      want = f64(x).T @ f64(gr)
      ws = torch.empty(L.ocnn_conv_dense_wgrad_rw_workspace_bytes(cin, cout), dtype=torch.uint8, device=DEV)
      got = []
      for transposed in (0, 1, 0):
        gw = torch.empty((cout, cin) if transposed else (cin, cout), dtype=dtype, device=DEV)
        _lib.check(L.ocnn_conv_dense_wgrad_rw(code, _lib.ptr(xd), _lib.ptr(gd), rows, cin, cout, transposed,
                                              _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
        got.append(gw.t() if transposed else gw)
        assert rel_err(got[-1], want) < TOL[dtype]
      assert torch.equal(got[0], got[1].contiguous()) and torch.equal(got[0], got[2])


def _gather_wide(x, rows_in, table, plan, w, cout, transposed, reverse, bias, occupancy=-1.0):
  """ocnn_conv_gather_wide through the C ABI (the Python layer picks it only for plans with
  enough reuse).  occupancy: the share of entries set as the entry point is told it (from 40 %
  down it leaves out the products of 32-row blocks without an entry in a slot)."""
  L = _lib.lib()
  rows, K = table.shape
  cin = x.shape[1]
  code = _lib.dtype_code(x)
  assert L.ocnn_conv_gather_wide_supported(code, rows_in, K, cin, cout, plan.umax)
  out = torch.empty((rows, cout), dtype=x.dtype, device=x.device)
  ws = torch.empty(K * (-(-cin // 64) * 64) * cout * 2, dtype=torch.uint8, device=x.device)   # whole 64-channel chunks
  _lib.check(L.ocnn_conv_gather_wide(
      code, _lib.ptr(x), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax,
      plan.total, occupancy, rows, K, _lib.ptr(w), cin, cout, int(transposed), int(reverse), _lib.ptr(bias),
      _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
  return out


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K,cin,cout', [(27, 128, 128), (27, 64, 256), (9, 192, 128), (8, 128, 384), (3, 256, 256),
                                        (1, 64, 128), (27, 96, 96), (27, 128, 96), (9, 96, 160), (3, 160, 224)])
def test_wide_gather_kernel(dtype, K, cin, cout):
  """Gather-GEMM for wide layers (weights streamed into registers, rows staged 64 input
  channels at a time), both output-channel widths per workgroup, channel counts that are
  odd multiples of 32 (half a chunk of input channels, idle waves on the output side), with
  bias, and the transposed + mirrored form, against the oracle.  The last input row is set
  to NaN where no table entry reads it: nothing beyond a row may leak into a result."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(7 * K + cin)
  for rows, rows_in in [(1000, 1000), (130, 150), (128 * 40 + 1, 3000)]:
    say('wide gather', dtype, K, cin, cout, rows, rows_in)
    table = _local_table(rows, rows_in - 1, K, g)        # the last input row is never read ..
    tg = table.to(DEV)
    plan = TilePlan(tg)
    t64 = table.numpy().astype(np.int64)
    x = torch.randn(rows_in, cin, generator=g).to(dtype)
    w = (torch.randn(K, cin, cout, generator=g) / (K * cin) ** 0.5).to(dtype)
    b = torch.randn(cout, generator=g).to(dtype)
    xn = x.clone()
    xn[-1] = float('nan')                                # .. and holds NaN
    got = _gather_wide(xn.to(DEV), rows_in, tg, plan, w.to(DEV), cout, False, False, b.to(DEV))
    want = C.forward_gemm(f64(x), f64(w), t64) + f64(b)
    assert rel_err(got, want) < TOL[dtype]
    if cin >= 96:                                        # the data gradient: cout -> cin
      gr = torch.randn(rows_in, cout, generator=g).to(dtype)
      got = _gather_wide(gr.to(DEV), rows_in, tg, plan, w.to(DEV), cin, True, True, None)
      want = C.forward_gemm(f64(gr), np.ascontiguousarray(f64(w)[::-1].transpose(0, 2, 1)), t64)
      assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize('K,cin,cout', [(27, 128, 128), (27, 128, 256), (9, 96, 160), (3, 256, 256), (8, 128, 128)])
def test_wide_gather_leaves_out_blocks_without_entries(K, cin, cout):
  """Told an occupancy of 40 % or less, the kernel for wide layers tests every (32-row block,
  slot) of a tile for entries and leaves the products of the empty ones out: tables where
  whole blocks, whole slots and whole tiles are empty, against the oracle and - bit for bit -
  against the same kernel without the test (occupancy unknown)."""
  from ocnn_amd.octree.octree import TilePlan
  dtype = torch.bfloat16
  g = torch.Generator().manual_seed(31 * K + cin)
  for rows, rows_in in [(128 * 9 + 77, 1400), (128 * 3, 500), (100, 90)]:
    say('wide gather with empty blocks', K, cin, cout, rows, rows_in)
    table = _local_table(rows, rows_in, K, g)
    blk = torch.arange(rows) // 32
    for k in range(K):
      table[(blk + k) % 3 == 0, k] = -1                  # a third of the (block, slot) units
    table[:, K // 2] = -1                                # a slot without entries
    if rows > 256:
      table[128:256] = -1                                # a tile without entries
      table[300:310, 0] = 5                              # (and a block with a few)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    t64 = table.numpy().astype(np.int64)
    x = torch.randn(rows_in, cin, generator=g).to(dtype)
    w = (torch.randn(K, cin, cout, generator=g) / (K * cin) ** 0.5).to(dtype)
    b = torch.randn(cout, generator=g).to(dtype)
    want = C.forward_gemm(f64(x), f64(w), t64) + f64(b)
    plain = _gather_wide(x.to(DEV), rows_in, tg, plan, w.to(DEV), cout, False, False, b.to(DEV))
    skipping = _gather_wide(x.to(DEV), rows_in, tg, plan, w.to(DEV), cout, False, False, b.to(DEV), occupancy=0.2)
    assert rel_err(plain, want) < TOL[dtype] and rel_err(skipping, want) < TOL[dtype]
    assert torch.equal(plain, skipping)
    gr = torch.randn(rows_in, cout, generator=g).to(dtype)
    if cin >= 96:
      a = _gather_wide(gr.to(DEV), rows_in, tg, plan, w.to(DEV), cin, True, True, None)
      c = _gather_wide(gr.to(DEV), rows_in, tg, plan, w.to(DEV), cin, True, True, None, occupancy=0.39)
      assert torch.equal(a, c)


def _gather_sparse(x, rows_in, table, plan, w, cout, transposed, reverse, bias):
  """ocnn_conv_gather_sparse through the C ABI (the Python layer picks it only for large,
  sparse tables)."""
  L = _lib.lib()
  rows, K = table.shape
  cin = x.shape[1]
  code = _lib.dtype_code(x)
  assert L.ocnn_conv_gather_sparse_supported(code, rows_in, K, cin, cout, plan.umax)
  import ctypes
  pp = plan.pairs()
  out = torch.empty((rows, cout), dtype=x.dtype, device=x.device)
  ws = torch.empty(L.ocnn_conv_gather_sparse_workspace_bytes(cin, cout), dtype=torch.uint8, device=x.device)
  _lib.check(L.ocnn_conv_gather_sparse(
      code, _lib.ptr(x), rows_in, _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax, plan.total,
      _lib.ptr(pp.cptr), _lib.ptr(pp.ent), pp.n_blocks, pp.max_blocks, _lib.ptr(pp.lists), pp.n_lists,
      ctypes.addressof(pp.group_bounds_host), rows, K, _lib.ptr(w), cin, cout, int(transposed), int(reverse),
      _lib.ptr(bias), _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
  return out


@pytest.mark.parametrize('K', [27, 8, 3, 1])
def test_pair_plan_lists(K):
  """The pair plan against its definition, from the tile plan's positions: per tile and list
  (slot, or rows r0 .. r1 - 1 of a heavy slot) the rows with a neighbour in ascending order,
  entry = position | r << 16, filled up to whole blocks of 16 with
  position 0 and r = 128."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(K)
  table = _local_table(128 * 9 + 50, 900, K, g, empty=0.8)
  if K > 2:
    table[:, 1] = -1
  if K == 27:
    table[:, 13] = torch.arange(table.shape[0], dtype=torch.int32).clamp_(max=899)
  plan = TilePlan(table.to(DEV))
  pp = plan.pairs()
  loc = plan.loc.cpu().numpy().astype(np.int64) & 0xffff      # (tiles, K, 128)
  tiles = loc.shape[0]
  lists = pp.lists.cpu().numpy()
  nl = pp.n_lists
  assert lists.tolist() == list(pp.lists_host)[:nl]
  if K in (27, 1):
    assert nl > K                                              # the full slot is cut by rows
  cptr = pp.cptr.cpu().numpy()
  ent = pp.ent.cpu().numpy().astype(np.int64) & 0xffffffff
  filler = 128 << 16
  at = 0
  most = 0
  for t in range(tiles):
    blocks = 0
    for j in range(nl):
      assert cptr[t * nl + j] == at
      k, r0, r1 = lists[j] & 255, (lists[j] >> 8) & 255, ((lists[j] >> 16) & 255) + 1
      rows = [r for r in range(r0, r1) if loc[t, k, r] > 0]
      want = [int(loc[t, k, r]) | (r << 16) for r in rows]
      want += [filler] * (-len(want) % 16)
      assert ent[16 * at:16 * at + len(want)].tolist() == want
      at += len(want) // 16
      blocks += len(want) // 16
    most = max(most, blocks)
  assert cptr[tiles * nl] == at == pp.n_blocks and most == pp.max_blocks


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K,cin,cout', [(27, 96, 96), (27, 128, 96), (27, 32, 64), (27, 64, 32), (9, 96, 128),
                                        (8, 128, 160), (8, 32, 32), (3, 64, 96), (1, 32, 32)])
def test_sparse_gather_kernel(dtype, K, cin, cout):
  """Gather-GEMM over the pair plan (blocks of 16 (row, neighbour) pairs per tile and slot,
  weights resident in registers, fp32 sums in LDS), at several occupancies incl. a table
  with empty slots and empty tiles, ragged row counts, with bias, and the transposed +
  mirrored form of the data gradient, against the oracle; twice, bit-identical.  The last
  input row holds NaN and is never read."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(11 * K + cin + cout)
  for rows, rows_in, empty in [(1000, 1000, 0.85), (130, 150, 0.5), (128 * 40 + 1, 3000, 0.9), (128 * 300 + 77, 40000, 0.8)]:
    say('sparse gather', dtype, K, cin, cout, rows, rows_in, empty)
    table = _local_table(rows, rows_in - 1, K, g, empty=empty)
    if K > 2:
      table[:, 1] = -1                                   # a slot without pairs
      table[256:384] = -1                                # a tile without pairs
    if K == 27:                                          # a slot with all the rows (it is cut into lists)
      table[:, 13] = torch.arange(rows, dtype=torch.int32).clamp_(max=rows_in - 2)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    t64 = table.numpy().astype(np.int64)
    x = torch.randn(rows_in, cin, generator=g).to(dtype)
    w = (torch.randn(K, cin, cout, generator=g) / (K * cin * (1 - empty)) ** 0.5).to(dtype)
    b = torch.randn(cout, generator=g).to(dtype)
    xn = x.clone()
    xn[-1] = float('nan')
    got = _gather_sparse(xn.to(DEV), rows_in, tg, plan, w.to(DEV), cout, False, False, b.to(DEV))
    again = _gather_sparse(xn.to(DEV), rows_in, tg, plan, w.to(DEV), cout, False, False, b.to(DEV))
    assert torch.equal(got, again)
    want = C.forward_gemm(f64(x), f64(w), t64) + f64(b)
    assert rel_err(got, want) < TOL[dtype]
    if cout <= 128:                                      # the data gradient: cout -> cin
      gr = torch.randn(rows_in, cout, generator=g).to(dtype)
      got = _gather_sparse(gr.to(DEV), rows_in, tg, plan, w.to(DEV), cin, True, True, None)
      want = C.forward_gemm(f64(gr), np.ascontiguousarray(f64(w)[::-1].transpose(0, 2, 1)), t64)
      assert rel_err(got, want) < TOL[dtype]


def _wgrad_sparse(x, g, table, plan, transposed):
  """ocnn_conv_wgrad_sparse through the C ABI."""
  import ctypes
  L = _lib.lib()
  rows, K = table.shape
  ca, cb = x.shape[1], g.shape[1]
  code = _lib.dtype_code(x)
  assert L.ocnn_conv_wgrad_sparse_supported(code, x.shape[0], rows, K, ca, cb, plan.umax)
  pp = plan.pairs()
  gw = torch.empty((K, cb, ca) if transposed else (K, ca, cb), dtype=x.dtype, device=x.device)
  ws = torch.empty(L.ocnn_conv_wgrad_sparse_workspace_bytes(rows, ca, cb), dtype=torch.uint8, device=x.device)
  _lib.check(L.ocnn_conv_wgrad_sparse(
      code, _lib.ptr(x), x.shape[0], ca, _lib.ptr(g), rows, cb, _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax,
      plan.total, _lib.ptr(pp.cptr), _lib.ptr(pp.ent), pp.n_blocks, ctypes.addressof(pp.lists_host),
      ctypes.addressof(pp.list_count_host), pp.n_lists, K, int(not transposed), _lib.ptr(gw), _lib.ptr(ws),
      ws.numel(), _lib.stream()))
  return gw


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K,ca,cb', [(27, 96, 96), (27, 128, 96), (27, 32, 64), (27, 64, 32), (27, 256, 32),
                                     (9, 96, 64), (8, 128, 96), (8, 32, 32), (3, 64, 96), (1, 32, 32)])
def test_sparse_wgrad_kernel(dtype, K, ca, cb):
  """Weight gradient over the pair plan (all slots of 32 x-channels in the registers of a
  workgroup, heavy slots cut into units, per-range sums added in a fixed order), at several
  occupancies incl. a slot and a tile without pairs and ragged row counts, both output
  layouts, against the oracle; twice, bit-identical.  The last x row holds NaN and is never
  read."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(5 * K + ca + cb)
  for rows, rows_in, empty in [(1000, 1000, 0.85), (130, 150, 0.5), (128 * 40 + 1, 3000, 0.9), (128 * 300 + 77, 40000, 0.8)]:
    say('sparse wgrad', dtype, K, ca, cb, rows, rows_in, empty)
    table = _local_table(rows, rows_in - 1, K, g, empty=empty)
    if K > 2:
      table[:, 1] = -1
      table[256:384] = -1
    if K == 27:
      table[:, 13] = torch.arange(rows, dtype=torch.int32).clamp_(max=rows_in - 2)   # a slot with all the rows
    tg = table.to(DEV)
    plan = TilePlan(tg)
    t64 = table.numpy().astype(np.int64)
    x = torch.randn(rows_in, ca, generator=g).to(dtype)
    gr = (torch.randn(rows, cb, generator=g) / (rows * (1 - empty)) ** 0.5).to(dtype)
    xn = x.clone()
    xn[-1] = float('nan')
    want = C.weight_gemm(f64(x), f64(gr), t64)
    for transposed in (False, True):
      got = _wgrad_sparse(xn.to(DEV), gr.to(DEV), tg, plan, transposed)
      again = _wgrad_sparse(xn.to(DEV), gr.to(DEV), tg, plan, transposed)
      assert torch.equal(got, again)
      assert rel_err(got, want.transpose(0, 2, 1) if transposed else want) < TOL[dtype]


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_layers_on_the_sparse_kernels(medium, dtype):
  """Whole layers (module forward + backward against the oracle) with the thresholds of the
  Python layer lowered so that the pair-plan kernels run on the test octree: 3x3x3 and axis
  kernels on non-empty nodes (gather, data gradient through the mirrored slots, weight
  gradient), 2x2x2 and 3x3x3 stride-2 conv / deconv (gathers over the table and its inverse,
  weight gradient over the inverse table)."""
  conv_mod = sys.modules['ocnn_amd.nn.octree_conv']
  keep = (conv_mod.SPARSE_MIN_ROWS, conv_mod.SPARSE_MAX_OCCUPANCY)
  conv_mod.SPARSE_MIN_ROWS, conv_mod.SPARSE_MAX_OCCUPANCY = 0, 1.0
  try:
    for kind, ks, stride, cin, cout in [('conv', [3], 1, 96, 96), ('conv', [3], 1, 128, 96), ('conv', [3, 3, 1], 1, 32, 96),
                                        ('conv', [2], 2, 96, 128), ('conv', [2], 2, 32, 64), ('deconv', [2], 2, 128, 96),
                                        ('deconv', [2], 2, 96, 32), ('deconv', [3], 1, 96, 64),
                                        ('conv', [3], 2, 64, 64), ('conv', [3], 2, 96, 32), ('deconv', [3], 2, 32, 96)]:
      depth = 6 if kind == 'deconv' and stride == 2 else 7
      say('layers on the sparse kernels', dtype, kind, ks, stride, cin, cout)
      errs = run_layer(kind, medium, depth, ks, stride, True, cin, cout, dtype)
      assert max(errs.values()) < TOL[dtype], (dtype, kind, ks, stride, cin, cout, errs)
  finally:
    conv_mod.SPARSE_MIN_ROWS, conv_mod.SPARSE_MAX_OCCUPANCY = keep


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_overflow_tiles_of_a_plan(dtype):
  """A few tiles with more distinct rows than the kernels on the plan take: the plan empties
  them and lists their rows, the Python layer runs those through the plan-free kernels;
  gather, mirrored data gradient and weight gradient of several kernels against the oracle."""
  from ocnn_amd.octree.octree import TilePlan
  conv_mod = sys.modules['ocnn_amd.nn.octree_conv']
  dw_mod = sys.modules['ocnn_amd.nn.octree_dwconv']
  g = torch.Generator().manual_seed(17)
  rows = rows_in = 128 * 60 + 31
  table = _local_table(rows, rows_in, 27, g, spread=40, empty=0.3)
  for t0 in (5, 33):                                       # two tiles that point all over the place
    table[128 * t0:128 * (t0 + 1)] = torch.randint(0, rows_in, (128, 27), generator=g).to(torch.int32)
  tg = table.to(DEV)
  plan = TilePlan(tg)
  assert plan.overflow_rows is not None and plan.overflow_rows.numel() == 256 and plan.umax <= TilePlan.CAP
  assert TilePlan(tg, cap=4096).overflow_rows is None
  t64 = table.numpy().astype(np.int64)
  for cin, cout in [(64, 64), (32, 32), (128, 128), (96, 96)]:
    say('overflow tiles', dtype, cin, cout)
    x = torch.randn(rows_in, cin, generator=g).to(dtype)
    w = (torch.randn(27, cin, cout, generator=g) / (19 * cin) ** 0.5).to(dtype)
    b = torch.randn(cout, generator=g).to(dtype)
    gr = (torch.randn(rows, cout, generator=g) / rows ** 0.5).to(dtype)
    got = conv_mod.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), cout, False, False, b.to(DEV), plan)
    assert rel_err(got, C.forward_gemm(f64(x), f64(w), t64) + f64(b)) < TOL[dtype]
    got = conv_mod.conv_gather(gr.to(DEV), rows_in, tg, w.to(DEV), cin, True, True, None, plan)
    want = C.forward_gemm(f64(gr), np.ascontiguousarray(f64(w)[::-1].transpose(0, 2, 1)), t64)
    assert rel_err(got, want) < TOL[dtype]
    got = conv_mod.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
    assert rel_err(got, C.weight_gemm(f64(x), f64(gr), t64)) < 2 * TOL[dtype]
  # depth-wise
  c = 64
  x = torch.randn(rows_in, c, generator=g).to(dtype)
  w = (torch.randn(27, 1, c, generator=g) / 19 ** 0.5).to(dtype)
  gr = (torch.randn(rows, c, generator=g) / rows ** 0.5).to(dtype)
  got = dw_mod.dw_gather(x.to(DEV), rows_in, tg, w.to(DEV), False, None, plan)
  valid = (t64 >= 0)[..., None]
  xg = f64(x)[np.maximum(t64, 0)] * valid                    # (rows, 27, c)
  assert rel_err(got, (xg * f64(w)[:, 0][None]).sum(1)) < TOL[dtype]
  got = dw_mod.dw_wgrad(x.to(DEV), gr.to(DEV), tg, plan)
  assert rel_err(got, (xg * f64(gr)[:, None, :]).sum(0)[:, None, :]) < 2 * TOL[dtype]


def test_sparse_gather_large_tiles():
  """Tiles near the staging limits of the pair-plan kernel (many distinct rows: one
  workgroup per CU, the wider row-number buffers) and the refusal beyond them."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(3)
  dtype = torch.bfloat16
  code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
  for cin, spread in [(96, 200), (128, 170), (32, 250)]:
    rows = rows_in = 6000
    table = _local_table(rows, rows_in, 27, g, spread=spread, empty=0.85)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    say('sparse gather, large tiles', cin, plan.umax)
    assert plan.umax > 256
    assert L.ocnn_conv_gather_sparse_supported(code, rows_in, 27, cin, 64, plan.umax)
    x = torch.randn(rows_in, cin, generator=g).to(dtype)
    w = (torch.randn(27, cin, 64, generator=g) / (4 * cin) ** 0.5).to(dtype)
    got = _gather_sparse(x.to(DEV), rows_in, tg, plan, w.to(DEV), 64, False, False, None)
    want = C.forward_gemm(f64(x), f64(w), table.numpy().astype(np.int64))
    assert rel_err(got, want) < TOL[dtype]
  assert not L.ocnn_conv_gather_sparse_supported(code, 6000, 27, 128, 64, 511)
  assert not L.ocnn_conv_gather_sparse_supported(code, 6000, 27, 96, 64, 600)
  assert not L.ocnn_conv_gather_sparse_supported(code, 6000, 27, 160, 64, 100)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K,ca,cb', [(27, 128, 128), (27, 64, 192), (9, 256, 64), (8, 128, 64), (3, 192, 128),
                                     (27, 96, 96), (27, 96, 128), (8, 160, 96), (3, 64, 96)])
def test_planned_wgrad_channel_blocks(dtype, K, ca, cb):
  """Weight gradient of layers with more than 64 channels: the planned kernel sums one
  64 x 64 block of channel pairs per workgroup."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(K + ca)
  for rows, rows_in in [(1000, 1000), (128 * 70 + 5, 5000)]:
    say('wgrad blocks', dtype, K, ca, cb, rows, rows_in)
    table = _local_table(rows, rows_in, K, g)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
    assert L.ocnn_conv_wgrad_planned_supported(code, rows_in, rows, K, ca, cb, plan.umax)
    x = torch.randn(rows_in, ca, generator=g).to(dtype)
    gr = torch.randn(rows, cb, generator=g).to(dtype)
    want = C.weight_gemm(f64(x), f64(gr), table.numpy().astype(np.int64))
    gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
    assert rel_err(gw, want) < TOL[dtype]
    gwt = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, True, plan)
    assert torch.equal(gwt, gw.transpose(1, 2).contiguous())
    assert torch.equal(gw, ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan))


@pytest.mark.parametrize('ch', [64, 32])
def test_planned_kernels_at_the_staging_limit(ch):
  """Tiles with exactly as many distinct rows as the persistent kernels stage (the last
  staged position is in use), and one more (the weight gradient then takes another kernel)."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(9)
  rows, K = 300, 27
  for distinct in (415, 416, 417):
    rows_in = 3 * distinct + 7
    table = torch.full((rows, K), -1, dtype=torch.int32)
    for t0 in range(0, rows, 128):                     # tile t draws from its own `distinct` rows
      n = min(128, rows - t0)
      pool = (torch.randperm(distinct, generator=g) + (t0 // 128) * distinct).to(torch.int32)
      e = pool[torch.randint(0, distinct, (n * K,), generator=g)]
      e[:distinct] = pool                              # every one of them at least once
      table[t0:t0 + n] = e[torch.randperm(n * K, generator=g)].reshape(n, K)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    assert plan.umax == distinct
    say('staging limit', ch, distinct, 'gather', L.ocnn_conv_gather_rw_supported(1, rows_in, K, ch, ch, plan.umax),
        'wgrad', L.ocnn_conv_wgrad_planned_supported(1, rows_in, rows, K, ch, ch, plan.umax))
    x = torch.randn(rows_in, ch, generator=g).half()
    gr = torch.randn(rows, ch, generator=g).half()
    w = (torch.randn(K, ch, ch, generator=g) / 30).half()
    t64 = table.numpy().astype(np.int64)
    out = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), ch, False, False, None, plan)
    assert rel_err(out, C.forward_gemm(f64(x), f64(w), t64)) < 2e-2
    gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
    assert rel_err(gw, C.weight_gemm(f64(x), f64(gr), t64)) < 2e-2


@pytest.mark.parametrize('K,ch', [(3, 32), (27, 32), (8, 32), (3, 64), (27, 64)])
def test_persistent_kernels_on_every_tile_count_per_workgroup(K, ch):
  """EVERY row of the persistent gather kernels against the plan-free kernel on tables whose
  workgroups get 3 m + 1, 3 m + 2 and 3 m tiles each (a ring of three tiles in LDS: the last one
  or two tiles of a range run outside the ring's loop).  The 32 -> 32 kernel waits for its loads
  by counting operations: the list entries the last tiles of a range load have no reader, the
  compiler dropped those loads, and the wait at the end of the tile before the last no longer
  covered the last tile's rows - a handful of wrong rows in some runs, found by the random
  layers at K = 3, where a tile is much shorter than a load."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(31 + K)
  wgs = torch.cuda.get_device_properties(0).multi_processor_count
  for per in (4, 5, 6, 11):
    rows = 128 * wgs * per - 37
    table = _local_table(rows, rows, K, g, spread=60, empty=0.4).to(DEV)
    plan = TilePlan(table)
    assert L.ocnn_conv_gather_rw_supported(2, rows, K, ch, ch, plan.umax)
    x = torch.randn(rows, ch, generator=g).bfloat16().to(DEV)
    w = (torch.randn(K, ch, ch, generator=g) / (K * ch) ** 0.5).bfloat16().to(DEV)
    want = ocnn_amd.nn.conv_gather(x, rows, table, w, ch, False, False, None, None).float()
    scale = float(want.abs().max())
    for rep in range(3):
      say('persistent gather, all rows', 'K', K, 'ch', ch, 'tiles per workgroup', per, 'run', rep)
      got = ocnn_amd.nn.conv_gather(x, rows, table, w, ch, False, False, None, plan).float()
      bad = ((got - want).abs().max(1).values > 2e-2 * scale).nonzero().view(-1)
      assert bad.numel() == 0, (K, ch, per, rep, bad[:8].tolist(), (bad // 128)[:8].tolist())


def test_other_planned_kernels_on_many_tile_counts():
  """The other kernels on the plan (weight gradient, wide gather, pair-plan gather and weight
  gradient, depth-wise gather and weight gradient) against the plan-free kernels on EVERY row,
  on tables of 4 .. 7 tiles per CU: ranges of tiles that end inside a ring of buffers, tails of
  every length."""
  from ocnn_amd.nn.octree_dwconv import dw_gather, dw_wgrad
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(5)
  wgs = torch.cuda.get_device_properties(0).multi_processor_count
  bf = torch.bfloat16

  def close(tag, got, want, per):
    got, want = got.float(), want.float()
    scale = float(want.abs().max())
    bad = ((got - want).abs().reshape(got.shape[0], -1).amax(1) > 2e-2 * scale).nonzero().view(-1)
    assert bad.numel() == 0, (tag, per, bad[:8].tolist())

  for per in (4, 5, 6, 7):
    rows = 128 * wgs * per - 61
    say('planned kernels, all rows, tiles per CU', per, 'rows', rows)
    table = _local_table(rows, rows, 27, g, spread=60, empty=0.4).to(DEV)
    plan = TilePlan(table)
    for ch in (32, 64):
      x = torch.randn(rows, ch, generator=g).to(bf).to(DEV)
      gr = torch.randn(rows, ch, generator=g).to(bf).to(DEV)
      close('weight gradient %d' % ch, ocnn_amd.nn.conv_wgrad(x, gr, table, False, plan),
            ocnn_amd.nn.conv_wgrad(x, gr, table, False, None), per)
    x = torch.randn(rows, 128, generator=g).to(bf).to(DEV)
    w = (torch.randn(27, 128, 128, generator=g) / (27 * 128) ** 0.5).to(bf).to(DEV)
    close('wide gather', _gather_wide(x, rows, table, plan, w, 128, False, False, None),
          ocnn_amd.nn.conv_gather(x, rows, table, w, 128, False, False, None, None), per)
    gr = torch.randn(rows, 128, generator=g).to(bf).to(DEV)
    close('weight gradient 128', ocnn_amd.nn.conv_wgrad(x, gr, table, False, plan),
          ocnn_amd.nn.conv_wgrad(x, gr, table, False, None), per)
    xd = torch.randn(rows, 64, generator=g).to(bf).to(DEV)
    wd = torch.randn(27, 1, 64, generator=g).to(bf).to(DEV)
    grd = torch.randn(rows, 64, generator=g).to(bf).to(DEV)
    plan.reuse = 10.0
    close('depth-wise gather', dw_gather(xd, rows, table, wd, False, None, plan), dw_gather(xd, rows, table, wd, False, None, None), per)
    close('depth-wise weight gradient', dw_wgrad(xd, grd, table, plan), dw_wgrad(xd, grd, table, None), per)
    sparse = _local_table(rows, rows, 27, g, spread=60, empty=0.85).to(DEV)
    splan = TilePlan(sparse)
    x = torch.randn(rows, 96, generator=g).to(bf).to(DEV)
    w = (torch.randn(27, 96, 96, generator=g) / (27 * 96 * 0.15) ** 0.5).to(bf).to(DEV)
    gr = torch.randn(rows, 96, generator=g).to(bf).to(DEV)
    close('pair-plan gather', _gather_sparse(x, rows, sparse, splan, w, 96, False, False, None),
          ocnn_amd.nn.conv_gather(x, rows, sparse, w, 96, False, False, None, None), per)
    close('pair-plan weight gradient', _wgrad_sparse(x, gr, sparse, splan, False),
          ocnn_amd.nn.conv_wgrad(x, gr, sparse, False, None), per)


@pytest.mark.parametrize('ch,empty,kernel', [(64, 0.3, 'GATHER_RW'), (128, 0.3, 'GATHER_WIDE'), (96, 0.85, 'GATHER_SPARSE')])
def test_tables_at_the_end_of_32_bit_offsets(ch, empty, kernel):
  """The kernels on the plan address their tensors with 32-bit byte offsets.  A table just
  under that range runs on them (the selection says so), one just over it on another
  kernel; either way the first, the last and 2000 random rows of output, data gradient and
  the whole weight gradient equal their fp64 definitions (rows near 2^32 bytes are where an
  offset that wraps would show)."""
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  K, dtype = 3, torch.bfloat16
  limit = 0xfff00000 // (ch * 2)                       # rows of `ch` bf16 channels in the range
  for rows, planned in ((limit - 4096 - 77, True), (limit + 4096 + 77, False)):
    say('tables at the end of 32-bit offsets:', ch, 'channels,', rows, 'rows,', kernel if planned else 'another kernel')
    g = torch.Generator(device=DEV).manual_seed(rows % 1000)
    base = torch.arange(rows, device=DEV).view(-1, 1)
    if kernel == 'GATHER_WIDE':                          # (that kernel is for tables whose tiles reuse their rows)
      table = (base + torch.arange(-1, K - 1, device=DEV).view(1, -1)).clamp_(0, rows - 1).to(torch.int32)
    else:
      table = (base + torch.randint(-40, 41, (rows, K), device=DEV, generator=g)).clamp_(0, rows - 1).to(torch.int32)
    table[torch.rand(rows, K, device=DEV, generator=g) < empty] = -1
    del base
    plan = TilePlan(table)
    code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
    took = L.ocnn_conv_gather_choose(code, rows, rows, K, ch, ch, 0, 1, plan.umax, plan.total, float(plan.occupancy),
                                     float(plan.reuse))
    assert (took == getattr(_lib, kernel)) == planned, (took, kernel)
    x = torch.randn(rows, ch, device=DEV, generator=g).to(dtype)
    gr = torch.randn(rows, ch, device=DEV, generator=g).to(dtype)
    w = (torch.randn(K, ch, ch, device=DEV, generator=g) / (K * ch) ** 0.5).to(dtype)
    sel = torch.cat([torch.arange(0, 1000, device=DEV), torch.arange(rows - 1000, rows, device=DEV),
                     torch.randint(0, rows, (2000,), device=DEV, generator=g)])
    ts = table[sel].long()

    def rows_of_definition(src, wk):                   # sum_k [t_ik >= 0] src[t_ik] @ wk(k), rows `sel`
      want = torch.zeros(sel.numel(), ch, dtype=torch.float64, device=DEV)
      for k in range(K):
        v = ts[:, k] >= 0
        want[v] += src[ts[v, k]].double() @ wk(k)
      return want

    out = ocnn_amd.nn.conv_gather(x, rows, table, w, ch, False, False, None, plan)
    assert rel_err(out[sel], rows_of_definition(x, lambda k: w[k].double()).cpu().numpy()) < TOL[dtype]
    del out
    # the mirrored form (data gradient of a symmetric table)
    out = ocnn_amd.nn.conv_gather(gr, rows, table, w, ch, True, True, None, plan)
    assert rel_err(out[sel], rows_of_definition(gr, lambda k: w[K - 1 - k].double().T).cpu().numpy()) < TOL[dtype]
    del out
    gw = ocnn_amd.nn.conv_wgrad(x, gr, table, False, plan)
    want = torch.empty(K, ch, ch, dtype=torch.float64, device=DEV)
    for k in range(K):
      v = torch.nonzero(table[:, k] >= 0).squeeze(1)
      acc = torch.zeros(ch, ch, dtype=torch.float64, device=DEV)
      for r0 in range(0, v.numel(), 1 << 22):            # (pieces: the fp64 copies of the rows are large)
        vv = v[r0:r0 + (1 << 22)]
        acc += x[table[vv, k].long()].double().T @ gr[vv].double()
      want[k] = acc
    assert rel_err(gw, want.cpu().numpy()) < TOL[dtype]
    del x, gr, table, plan, gw, want
    torch.cuda.empty_cache()


@pytest.mark.parametrize('kernel', ['333', '331', '313', '133', '311', '131', '113'])
def test_stride2_data_gradient_in_block_form(medium, kernel):
  """backward_gemm of the stride-2 layers over all nodes as a 2x2x2 stride-1 gather over the
  non-empty coarse nodes with block weights: the path is taken (64 and 96 channels, f16 and bf16,
  with and without bias) and gives the oracle's scatter over the layer's own table, rows of all
  fine nodes; fp32 and 32 output channels take the inverse table and give the same.  Likewise
  the weight gradient on the planned kernel over the mirror image of that table."""
  import importlib
  OC = importlib.import_module('ocnn_amd.nn.octree_conv')
  o, ref, depth = medium.gpu, medium.ref, 7
  ks = [int(c) for c in kernel]
  g = torch.Generator().manual_seed(17)
  table = ref.get_neigh(depth, kernel, 2, False).astype(np.int64)
  P, fine = table.shape[0], int(ref.nnum[depth])
  assert fine == 8 * P
  for cin, cout, dtype, blocks in ((64, 64, torch.bfloat16, True), (96, 64, torch.float16, True), (32, 128, torch.bfloat16, True),
                                   (64, 32, torch.bfloat16, False), (64, 64, torch.float32, False)):
    eng = OC._OctreeConv(cin, cout, ks, 2, False, int(2e8))
    eng.setup(o, depth)
    assert eng.block_children and eng.coarse_depth == depth - 1
    grad = torch.randn(P, cout, generator=g).to(dtype)
    w = (torch.randn(len(table[0]), cin, cout, generator=g) / (len(table[0]) * cout) ** 0.5).to(dtype)
    b = torch.randn(cin, generator=g).to(dtype)
    want = C.backward_gemm(f64(grad), f64(w), table, fine)
    say('stride-2 data gradient', kernel, cin, cout, dtype, 'block form' if blocks else 'inverse table')
    got = eng._backward_blocks(grad.to(DEV), w.to(DEV), None)
    assert (got is not None) == blocks
    tol = 1e-4 if dtype == torch.float32 else TOL[dtype]
    if blocks:
      assert got.shape == (fine, cin) and rel_err(got, want) < tol
      assert rel_err(eng._backward_blocks(grad.to(DEV), w.to(DEV), b.to(DEV)), want + f64(b)) < tol
    assert rel_err(eng.backward_gemm(grad.to(DEV), w.to(DEV)), want) < tol
    # the weight gradient on the planned kernel over the mirror table, or as before
    x = torch.randn(fine, cin, generator=g).to(dtype)
    want = C.weight_gemm(f64(x), f64(grad), table)
    gw = eng._weight_blocks(x.to(DEV), grad.to(DEV), False)
    assert (gw is not None) == (cout >= 64), (cin, cout, dtype)       # (fp32: as bf16 pieces on the same kernel)
    if gw is not None:
      assert gw.shape == want.shape and rel_err(gw, want) < tol
      assert torch.equal(eng._weight_blocks(x.to(DEV), grad.to(DEV), True), gw.transpose(1, 2).contiguous())
    assert rel_err(eng.weight_gemm(x.to(DEV), grad.to(DEV)), want) < tol


def test_planned_kernels_non_finite_rows():
  """Rows past the end of the table and empty entries must not pick up values of
  staged rows: NaN / Inf rows that no valid entry refers to stay out of the result."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(77)
  rows, rows_in, K = 200, 260, 27
  table = _local_table(rows, rows_in - 4, K, g)            # the last 4 input rows are never referenced
  x = torch.randn(rows_in, 64, generator=g).half()
  x[-4:] = float('nan')
  x[0] = float('inf')
  table[table == 0] = -1                                    # nor is row 0
  gr = torch.randn(rows, 64, generator=g).half()
  w = (torch.randn(K, 64, 64, generator=g) / 40).half()
  tg = table.to(DEV)
  plan = TilePlan(tg)
  out = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), 64, False, False, None, plan)
  gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
  assert torch.isfinite(out).all() and torch.isfinite(gw).all()


def test_planned_kernels_fall_back_on_large_tiles():
  """A tile with more distinct rows than the persistent kernels stage: the entry points
  report it and the Python layer takes the other kernels (same results)."""
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(5)
  rows, rows_in, K = 500, 50000, 27
  table = torch.randint(0, rows_in, (rows, K), generator=g, dtype=torch.int32)
  tg = table.to(DEV)
  plan = TilePlan(tg)
  assert plan.umax > 512
  L = _lib.lib()
  assert not L.ocnn_conv_gather_rw_supported(1, rows_in, K, 64, 64, plan.umax)
  assert not L.ocnn_conv_wgrad_planned_supported(1, rows_in, rows, K, 64, 64, plan.umax)
  x = torch.randn(rows_in, 64, generator=g).half()
  gr = torch.randn(rows, 64, generator=g).half()
  w = (torch.randn(K, 64, 64, generator=g) / 40).half()
  t64 = table.numpy().astype(np.int64)
  out = ocnn_amd.nn.conv_gather(x.to(DEV), rows_in, tg, w.to(DEV), 64, False, False, None, plan)
  assert rel_err(out, C.forward_gemm(f64(x), f64(w), t64)) < 2e-2
  gw = ocnn_amd.nn.conv_wgrad(x.to(DEV), gr.to(DEV), tg, False, plan)
  assert rel_err(gw, C.weight_gemm(f64(x), f64(gr), t64)) < 2e-2


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('K,ch', [(27, 64), (27, 192), (9, 128), (8, 64), (3, 128)])
def test_dwconv_planned_kernels(dtype, K, ch):
  """Depth-wise kernels on the tile plan (rows staged in LDS): gather with bias, with mirrored
  slots, and the weight gradient (the slot counts it is built for), against the oracle."""
  from ocnn_amd.nn.octree_dwconv import dw_gather, dw_wgrad
  from ocnn_amd.octree.octree import TilePlan
  L = _lib.lib()
  g = torch.Generator().manual_seed(11 * K + ch)
  code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
  for rows, rows_in in [(1000, 1000), (130, 150), (128 * 50 + 7, 4000)]:
    say('dwconv planned', dtype, K, ch, rows, rows_in)
    table = _local_table(rows, rows_in, K, g)
    tg = table.to(DEV)
    plan = TilePlan(tg)
    plan.reuse = 10.0                                    # take the staged kernels whatever the table's reuse
    t64 = table.numpy().astype(np.int64)
    assert L.ocnn_dwconv_gather_planned_supported(code, rows_in, K, ch, plan.umax)
    x = torch.randn(rows_in, ch, generator=g).to(dtype)
    w = torch.randn(K, 1, ch, generator=g).to(dtype)
    b = torch.randn(ch, generator=g).to(dtype)
    gr = torch.randn(rows, ch, generator=g).to(dtype)
    got = dw_gather(x.to(DEV), rows_in, tg, w.to(DEV), False, b.to(DEV), plan)
    assert rel_err(got, C.dw_forward(f64(x), f64(w), t64) + f64(b)) < TOL[dtype]
    got = dw_gather(x.to(DEV), rows_in, tg, w.to(DEV), True, None, plan)
    assert rel_err(got, C.dw_forward(f64(x), f64(w)[::-1], t64)) < TOL[dtype]
    if K in (27, 9, 8, 3):
      assert L.ocnn_dwconv_wgrad_planned_supported(code, rows_in, rows, K, ch, plan.umax)
    gw = dw_wgrad(x.to(DEV), gr.to(DEV), tg, plan)
    assert rel_err(gw, C.dw_weight(f64(x), f64(gr), t64)) < TOL[dtype]
    assert torch.equal(gw, dw_wgrad(x.to(DEV), gr.to(DEV), tg, plan))


def test_dwconv_planned_non_finite_values_stay_in_their_group_of_four():
  """The planned depth-wise gather multiplies on the 4x4x4 matrix instruction with diag(w) as one
  operand, so 0 x inf of one channel reaches the other three channels of its group of four as
  NaN; the per-channel kernel (and the reference) keeps it in its own channel.  Fixed here: an
  infinite input value makes non-finite outputs only in rows that read its row, and there only
  in the channels 4 * (c / 4) .. + 3; every other value equals the result on the finite input."""
  from ocnn_amd.nn.octree_dwconv import dw_gather
  from ocnn_amd.octree.octree import TilePlan
  g = torch.Generator().manual_seed(99)
  K, ch, rows = 27, 64, 1000
  table = _local_table(rows, rows, K, g)
  tg = table.to(DEV)
  plan = TilePlan(tg)
  plan.reuse = 10.0
  for dtype in (torch.float16, torch.bfloat16):
    x = torch.randn(rows, ch, generator=g).to(dtype).to(DEV)
    w = torch.randn(K, 1, ch, generator=g).to(dtype).to(DEV)
    clean = dw_gather(x, rows, tg, w, False, None, plan)
    bad_row, bad_ch = 321, 13
    x2 = x.clone()
    x2[bad_row, bad_ch] = float('inf')
    got = dw_gather(x2, rows, tg, w, False, None, plan)
    readers = (tg == bad_row).any(1)                       # rows that gather the bad row
    group = torch.zeros(ch, dtype=torch.bool, device=DEV)
    group[4 * (bad_ch // 4):4 * (bad_ch // 4) + 4] = True
    touched = readers.unsqueeze(1) & group.unsqueeze(0)
    assert bool(readers.any())
    assert torch.equal(got[~touched], clean[~touched])
    assert not bool(torch.isfinite(got[readers][:, bad_ch]).any())     # its own channel: inf (or NaN), as it must be
    # the plan-free kernel keeps the value in its channel
    plain = dw_gather(x2, rows, tg, w, False, None, None)
    own = readers.unsqueeze(1) & (torch.arange(ch, device=DEV) == bad_ch).unsqueeze(0)
    assert bool(torch.isfinite(plain[~own]).all())


def test_dwconv_all_slot_kernels(medium):
  """Depth-wise kernels that keep all slots of a row in one thread (power-of-two channel
  counts), every slot count, fp32 and 16-bit, against the oracle."""
  for dtype in (torch.float32, torch.float16, torch.bfloat16):
    for ks, stride, ne, C, depth in [([3], 1, False, 32, 6), ([3], 1, True, 64, 7), ([2], 2, False, 16, 7),
                                     ([2], 2, True, 8, 6), ([3, 1, 3], 1, False, 128, 5),
                                     ([1, 1, 3], 1, True, 4, 6)]:
      say('dwconv', dtype, ks, stride, ne, C, depth)
      errs = run_layer('dwconv', medium, depth, ks, stride, ne, C, C, dtype)
      assert max(errs.values()) < TOL[dtype], (dtype, ks, stride, ne, C, errs)


def test_pad_depad_wide_rows(small):
  """16-byte-per-thread pad / depad (row size a multiple of 16 bytes)."""
  d = 5
  for dt, ch in ((torch.float32, 8), (torch.float16, 64), (torch.bfloat16, 24)):
    x = torch.randn(int(small.ref.nnum_nempty[d]), ch).to(dt).to(DEV)
    p = octree_pad(x, small.gpu, d, val=-2.5)
    assert np.array_equal(f64(p), C.octree_pad(f64(x), small.ref, d, -2.5))
    y = torch.randn(int(small.ref.nnum[d]), ch).to(dt).to(DEV)
    assert np.array_equal(f64(octree_depad(y, small.gpu, d)), C.octree_depad(f64(y), small.ref, d))


def test_odd_channels_on_large_layers(medium):
  """Channel counts the MFMA kernels do not take are zero-padded once the layer is large
  (first and last layers of a network: 4 -> 32, 32 -> 10 ...)."""
  conv_mod = sys.modules['ocnn_amd.nn.octree_conv']
  assert rows_of(medium.ref, 7, False) >= conv_mod.PAD_MIN_ROWS
  for dtype in (torch.float32, torch.bfloat16):
    for kind, ks, stride, ne, cin, cout in [('conv', [3], 1, False, 4, 32), ('conv', [3], 1, False, 32, 10),
                                            ('conv', [2], 2, False, 5, 7), ('deconv', [2], 2, False, 12, 6),
                                            ('conv', [3], 1, True, 3, 3)]:
      depth = 6 if kind == 'deconv' else 7
      say('padded channels', dtype, kind, ks, stride, ne, cin, cout)
      errs = run_layer(kind, medium, depth, ks, stride, ne, cin, cout, dtype)
      assert max(errs.values()) < TOL[dtype], (dtype, kind, ks, stride, ne, cin, cout, errs)


def test_group_conv_is_a_block_diagonal_conv(small):
  """OctreeGroupConv (ocnn/nn/octree_gconv.py): its output equals the oracle's convolution
  with the block-diagonal weights put together from the per-group layers."""
  from ocnn_amd.nn import OctreeGroupConv
  depth, cin, cout, group = 5, 12, 18, 3
  g = torch.Generator().manual_seed(21)
  mod = OctreeGroupConv(cin, cout, [3], 1, nempty=True, use_bias=True, group=group).to(DEV)
  x = torch.randn(rows_of(small.ref, depth, True), cin, generator=g)
  out = mod(x.to(DEV), small.gpu, depth)
  w = np.zeros((27, cin, cout))
  b = np.zeros(cout)
  ci, co = cin // group, cout // group
  for i, conv in enumerate(mod.convs):
    w[:, i * ci:(i + 1) * ci, i * co:(i + 1) * co] = f64(conv.weights)
    b[i * co:(i + 1) * co] = f64(conv.bias)
  want = C.conv_layer(small.ref, f64(x), w, depth, [3, 3, 3], 1, True, bias=b)
  assert rel_err(out, want) < 1e-4


@pytest.mark.parametrize('first', [0, 40, 80])
def test_random_shapes_through_the_dispatch(first):
  """Random tables (local or scattered entries, 5 % .. 100 % set, ragged row counts, a stretch
  of empty rows), channel counts (multiples of 32, and 4 / 8 / 10 / 16 / 48) and slot counts
  through conv_gather / conv_wgrad, which pick the kernel per shape and plan: output, the
  transposed-weight form and both weight-gradient layouts against the oracle."""
  from ocnn_amd.octree.octree import TilePlan
  chans = [32, 64, 96, 128, 160, 192, 256, 48, 16, 8, 4, 10, 384]
  for case in range(first, first + 40):
    rng = np.random.default_rng(case)
    dtype = [torch.float16, torch.bfloat16][case % 2]
    K = int(rng.choice([1, 3, 8, 9, 27]))
    cin, cout = int(rng.choice(chans)), int(rng.choice(chans))
    rows = int(rng.choice([1, 5, 127, 129, 1000, 5000, 20000, 33000, 70000]))
    rows_in = int(rng.choice([1, 7, 300, 5000, 20000, 40000])) if rng.random() < 0.5 else rows
    p = float(rng.choice([0.05, 0.15, 0.3, 0.6, 1.0]))
    local = rng.random() < 0.7
    if local:                                   # entries near the row: plans with reuse
      t = (np.arange(rows)[:, None] * rows_in // max(rows, 1) + rng.integers(-40, 41, size=(rows, K))) % rows_in
    else:
      t = rng.integers(0, rows_in, size=(rows, K))
    t = np.where(rng.random((rows, K)) < p, t, -1).astype(np.int32)
    if rng.random() < 0.3 and rows > 200:
      t[100:200] = -1
    x = torch.from_numpy(rng.standard_normal((rows_in, cin)).astype(np.float32)).to(dtype)
    w = torch.from_numpy((rng.standard_normal((K, cin, cout)) / np.sqrt(K * cin)).astype(np.float32)).to(dtype)
    b = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to(dtype) if rng.random() < 0.5 else None
    gr = torch.from_numpy(rng.standard_normal((rows, cout)).astype(np.float32)).to(dtype)
    use_plan = rng.random() < 0.8
    say('random case', case, dtype, 'K', K, cin, '->', cout, 'rows', rows, 'rows_in', rows_in, 'set', p,
        'local', local, 'plan', use_plan, 'bias', b is not None)
    td = torch.from_numpy(t).to(DEV)
    plan = TilePlan(td) if use_plan else None
    t64 = t.astype(np.int64)
    xd, wd, gd = x.to(DEV), w.to(DEV), gr.to(DEV)
    want = C.forward_gemm(f64(x), f64(w), t64)
    out = ocnn_amd.nn.conv_gather(xd, rows_in, td, wd, cout, False, False, None if b is None else b.to(DEV), plan)
    assert rel_err(out, want + (0 if b is None else f64(b))) < TOL[dtype]
    out = ocnn_amd.nn.conv_gather(xd, rows_in, td, w.transpose(1, 2).contiguous().to(DEV), cout, True, False,
                                  None, plan)
    assert rel_err(out, want) < TOL[dtype]
    want = C.weight_gemm(f64(x), f64(gr), t64)
    assert rel_err(ocnn_amd.nn.conv_wgrad(xd, gd, td, False, plan), want) < TOL[dtype]
    assert rel_err(ocnn_amd.nn.conv_wgrad(xd, gd, td, True, plan).transpose(1, 2), want) < TOL[dtype]


def test_random_large_tables_planned_against_plan_free():
  """Large random tables (80 k .. 1.5 M rows, 3 .. 27 slots, 32 .. 256 channels, 5 % .. 100 % of the
  entries set, narrow to wide neighbourhoods): the kernels the selection takes with a plan
  against the plan-free kernels on EVERY row of output and mirrored gather, on the weight
  gradient, and (64-channel multiples) on the depth-wise pair.  No oracle at these sizes: the
  plan-free kernels are held to it elsewhere; this is about row ranges, tails and tile counts
  per workgroup that small tables do not reach.  3 x OCNN_TEST_CASES cases (default 120) from
  OCNN_TEST_FIRST on."""
  from ocnn_amd.nn.octree_dwconv import dw_gather, dw_wgrad
  from ocnn_amd.octree.octree import TilePlan
  chans = [32, 64, 96, 128, 160, 192, 256]
  cases = random_cases(40)
  for case in range(3 * cases.start, 3 * cases.stop):
    rng = np.random.default_rng(case)
    g = torch.Generator(device=DEV).manual_seed(case)
    dtype = [torch.float16, torch.bfloat16][case % 2]
    K = int(rng.choice([3, 8, 9, 27, 27, 27]))
    cin = int(rng.choice(chans))
    cout = cin if rng.random() < 0.6 else int(rng.choice(chans))
    rows = int(rng.integers(80_000, 1_500_000))
    rows_in = rows if rng.random() < 0.6 else int(rng.integers(40_000, 1_500_000))
    p = float(rng.choice([0.05, 0.1, 0.15, 0.25, 0.35, 0.6, 1.0]))
    spread = int(rng.choice([3, 10, 40, 150]))
    base = (torch.arange(rows, device=DEV, dtype=torch.float64) * (rows_in / rows)).long().view(-1, 1)
    t = (base + torch.randint(-spread, spread + 1, (rows, K), device=DEV, generator=g)).clamp_(0, rows_in - 1).to(torch.int32)
    t[torch.rand(rows, K, device=DEV, generator=g) >= p] = -1
    plan = TilePlan(t)
    x = torch.randn(rows_in, cin, device=DEV, generator=g).to(dtype)
    w = (torch.randn(K, cin, cout, device=DEV, generator=g) / (K * cin * p) ** 0.5).to(dtype)
    gr = torch.randn(rows, cout, device=DEV, generator=g).to(dtype)
    tag = 'large random table %d: %s K %d %d -> %d rows %d rows_in %d set %.2f spread %d, %d distinct rows a tile at most' % (
        case, str(dtype)[6:], K, cin, cout, rows, rows_in, p, spread, plan.umax)
    say(tag)

    def close(name, got, want):
      got, want = got.float(), want.float()
      scale = float(want.abs().max()) + 1e-30
      d = (got - want).abs().reshape(got.shape[0], -1).amax(1)
      wrong = (d > 2e-2 * scale).nonzero().view(-1)
      assert wrong.numel() == 0, (tag, name, wrong.numel(), wrong[:8].tolist(), float(d.max()) / scale)

    close('gather', ocnn_amd.nn.conv_gather(x, rows_in, t, w, cout, False, False, None, plan),
          ocnn_amd.nn.conv_gather(x, rows_in, t, w, cout, False, False, None, None))
    if rows_in == rows:
      close('mirrored gather', ocnn_amd.nn.conv_gather(gr, rows, t, w, cin, True, True, None, plan),
            ocnn_amd.nn.conv_gather(gr, rows, t, w, cin, True, True, None, None))
    close('weight gradient', ocnn_amd.nn.conv_wgrad(x, gr, t, False, plan), ocnn_amd.nn.conv_wgrad(x, gr, t, False, None))
    if cin == cout and cin % 64 == 0 and case % 3 == 0:
      wd = torch.randn(K, 1, cin, device=DEV, generator=g).to(dtype)
      close('depth-wise gather', dw_gather(x, rows_in, t, wd, False, None, plan), dw_gather(x, rows_in, t, wd, False, None, None))
      close('depth-wise weight gradient', dw_wgrad(x, gr, t, plan), dw_wgrad(x, gr, t, None))
    del x, w, gr, t, plan, base


def test_random_sizes_of_the_dense_kernels_against_torch():
  """The persistent one-slot kernels (the form of the 2x2x2 stride-2 layers) on random row
  counts up to 2 M, operands read and results written through a row index, against torch's
  matmul in fp32 on every row.  OCNN_TEST_CASES cases (default 40) from OCNN_TEST_FIRST on."""
  L = _lib.lib()
  for case in random_cases(40):
    rng = np.random.default_rng(case)
    g = torch.Generator(device=DEV).manual_seed(case)
    dtype = [torch.float16, torch.bfloat16][case % 2]
    code = _lib.dtype_code(torch.zeros(1, dtype=dtype))
    cin, cout = int(rng.choice([64, 128, 256, 512])), int(rng.choice([128, 256, 384, 512]))
    rows = int(rng.integers(1000, 2_000_000)) if rng.random() < 0.8 else int(rng.integers(1, 3000))
    n_all = rows + int(rng.integers(0, rows + 10))
    say('dense kernels, random sizes', case, dtype, cin, cout, 'rows', rows, 'of', n_all)
    x_all = torch.randn(n_all, cin, device=DEV, generator=g).to(dtype)
    gr_all = torch.randn(n_all, cout, device=DEV, generator=g).to(dtype)
    idx = torch.sort(torch.randperm(n_all, device=DEV, generator=g)[:rows]).values.to(torch.int32)
    w = (torch.randn(cin, cout, device=DEV, generator=g) / cin ** 0.5).to(dtype)
    b = torch.randn(cout, device=DEV, generator=g).to(dtype)
    xc = x_all[:rows].contiguous()

    def close(name, got, want):
      got, want = got.float(), want.float()
      scale = float(want.abs().max()) + 1e-30
      d = (got - want).abs().reshape(got.shape[0], -1).amax(1)
      wrong = (d > 2e-2 * scale).nonzero().view(-1)
      assert wrong.numel() == 0, (case, name, wrong.numel(), wrong[:8].tolist(), float(d.max()) / scale)

    if L.ocnn_conv_dense_rw_supported(code, n_all, cin, cout):
      ws = torch.empty(cin * cout * 2, dtype=torch.uint8, device=DEV)
      out = torch.empty(rows, cout, dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_rw_indexed(code, _lib.ptr(x_all), n_all, _lib.ptr(idx), rows, _lib.ptr(w), cin, cout, 0,
                                              _lib.ptr(b), _lib.ptr(out), rows, None, _lib.ptr(ws), ws.numel(), _lib.stream()))
      close('rows read through an index', out, x_all[idx.long()].float() @ w.float() + b.float())
      out = torch.zeros(n_all, cout, dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_rw_indexed(code, _lib.ptr(xc), rows, None, rows, _lib.ptr(w), cin, cout, 0,
                                              _lib.ptr(b), _lib.ptr(out), n_all, _lib.ptr(idx), _lib.ptr(ws), ws.numel(),
                                              _lib.stream()))
      want = torch.zeros(n_all, cout, device=DEV)
      want[idx.long()] = xc.float() @ w.float() + b.float()
      close('rows written through an index', out, want)
    if L.ocnn_conv_dense_wgrad_rw_supported(code, n_all, cin, cout):
      ws = torch.empty(L.ocnn_conv_dense_wgrad_rw_workspace_bytes(cin, cout), dtype=torch.uint8, device=DEV)
      gw = torch.empty(cin, cout, dtype=dtype, device=DEV)
      _lib.check(L.ocnn_conv_dense_wgrad_rw_indexed(code, _lib.ptr(xc), rows, None, _lib.ptr(gr_all), n_all, _lib.ptr(idx), rows,
                                                    cin, cout, 0, _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
      close('weight gradient, g through an index', gw, xc.float().T @ gr_all[idx.long()].float())
    del x_all, gr_all, idx, xc


def test_random_layers_vs_oracle():
  """Random module configurations (conv / deconv / depth-wise, all eight kernel shapes, both
  strides, all or non-empty nodes, channel counts incl. 4 / 10 / 16 / 48, f16 / bf16 / fp32, with
  and without bias) on octrees of depth 5 to 8: forward and all gradients against the oracle.
  OCNN_TEST_CASES sets the number of cases (default 48), OCNN_TEST_FIRST the first one."""
  octs = [(5, 2, 3000, 1), (6, 3, 8000, 2), (7, 2, 30000, 3), (7, 1, 60000, 4), (8, 2, 50000, 5)]
  kerns = ['333', '222', '311', '131', '113', '331', '313', '133']
  chans = [32, 64, 96, 128, 48, 16, 4, 10, 160, 256]
  pairs = {}
  for case in random_cases(48):
    rng = np.random.default_rng(case)
    kind = ['conv', 'deconv', 'dwconv'][int(rng.integers(0, 3))]
    depth, batch, n, seed = octs[int(rng.integers(0, len(octs)))]
    kern = kerns[int(rng.integers(0, 8))] if rng.random() < 0.5 else ['333', '222'][int(rng.integers(0, 2))]
    stride = int(rng.choice([1, 2])) if kern != '222' else 2
    ne = bool(rng.integers(0, 2))
    cin, cout = int(rng.choice(chans)), int(rng.choice(chans))
    dtype = [torch.float16, torch.bfloat16, torch.float32][int(rng.choice([0, 1, 1, 0, 2]))]
    if dtype == torch.float32:
      cin, cout = min(cin, 32), min(cout, 32)
    if kind == 'dwconv':
      cout = cin
    if (depth, batch) not in pairs:
      pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, batch, seed, n=n)
      pairs[(depth, batch)] = Pair(pts, nrm, bid if batch > 1 else None, depth, 2, batch)
    d = depth - 1 if (kind == 'deconv' and stride == 2) else depth
    bias = bool(rng.integers(0, 2))
    say('random layer', case, kind, kern, 'stride', stride, 'nempty', ne, cin, '->', cout, dtype, 'depth', d,
        'of', depth, 'batch', batch, 'bias', bias)
    errs = run_layer(kind, pairs[(depth, batch)], d, [int(c) for c in kern], stride, ne, cin, cout, dtype,
                     seed=case, use_bias=bias)
    assert max(errs.values()) < TOL[dtype], (case, errs)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_empty_inputs(dtype):
  """Tables without rows, and tables whose entries are all -1 over an input without rows: empty
  outputs, resp. zeros (+ bias), and zero weight gradients, with and without a plan."""
  from ocnn_amd.octree.octree import TilePlan
  for K, cin, cout in [(27, 64, 64), (27, 96, 96), (8, 128, 128), (1, 64, 128), (27, 5, 7)]:
    say('empty inputs', dtype, K, cin, cout)
    w = torch.randn(K, cin, cout, device=DEV).to(dtype)
    b = torch.randn(cout, device=DEV).to(dtype)
    t0 = torch.empty((0, K), dtype=torch.int32, device=DEV)
    x = torch.randn(10, cin, device=DEV).to(dtype)
    g0 = torch.empty((0, cout), device=DEV).to(dtype)
    t1 = torch.full((300, K), -1, dtype=torch.int32, device=DEV)
    x0 = torch.empty((0, cin), device=DEV).to(dtype)
    g1 = torch.randn(300, cout, device=DEV).to(dtype)
    for plan0, plan1 in [(None, None), (TilePlan(t0), TilePlan(t1))]:
      out = ocnn_amd.nn.conv_gather(x, 10, t0, w, cout, False, False, b, plan0)
      assert tuple(out.shape) == (0, cout)
      gw = ocnn_amd.nn.conv_wgrad(x, g0, t0, False, plan0)
      assert tuple(gw.shape) == (K, cin, cout) and not gw.any()
      out = ocnn_amd.nn.conv_gather(x0, 0, t1, w, cout, False, False, b, plan1)
      assert torch.equal(out, b.view(1, -1).expand(300, cout))
      gw = ocnn_amd.nn.conv_wgrad(x0, g1, t1, True, plan1)
      assert tuple(gw.shape) == (K, cout, cin) and not gw.any()


@pytest.mark.parametrize('kind,ks,stride,nempty,cin,cout', [
    ('conv', [3], 1, False, 64, 64), ('conv', [3], 1, True, 96, 96), ('conv', [2], 2, False, 64, 128),
    ('deconv', [2], 2, False, 128, 64), ('dwconv', [3], 1, False, 64, 64)])
def test_layers_replay_from_a_hip_graph(medium, kind, ks, stride, nempty, cin, cout):
  """The library only launches kernels on the caller's stream (no allocation, memset, copy or
  synchronisation of its own), so forward + backward of a layer can be captured in a HIP graph once
  its plans exist: three replays, with eager work and synchronisations in between, give the bits
  of the eager run."""
  depth, dtype = 7, torch.bfloat16
  o = medium.gpu
  say('hip graph', kind, ks, stride, nempty, cin, cout)
  g = torch.Generator().manual_seed(5)
  if kind == 'conv':
    mod = OctreeConv(cin, cout, ks, stride, nempty, use_bias=True)
  elif kind == 'deconv':
    mod = OctreeDeconv(cin, cout, ks, stride, nempty, use_bias=True)
  else:
    mod = OctreeDWConv(cin, ks, stride, nempty, use_bias=True)
  mod = mod.to(DEV).to(dtype)
  d_in = depth - 1 if kind == 'deconv' else depth
  rows = int(o.nnum_nempty[d_in] if nempty else o.nnum[d_in])
  x = torch.randn(rows, cin, generator=g).to(dtype).to(DEV).requires_grad_()
  params = [x] + list(mod.parameters())

  def step():
    for p in params:
      p.grad = None
    out = mod(x, o, d_in)
    out.backward(gout)
    return out

  gout = torch.randn(mod(x, o, d_in).shape, generator=g).to(dtype).to(DEV)
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    for _ in range(2):
      out = step()                                    # plans, tables and workspaces exist from here on
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  want = [out.detach().clone()] + [p.grad.clone() for p in params]
  del out                              # no autograd graph of the eager runs (and its stream) stays alive
  graph = torch.cuda.CUDAGraph()
  for p in params:
    p.grad = None
  with torch.cuda.graph(graph):
    out_g = mod(x, o, d_in)
    out_g.backward(gout)
  for replay in range(3):
    out_g.detach().zero_()
    for p in params:
      p.grad.zero_()
    (torch.randn(1000, 64, device=DEV) @ torch.randn(64, 64, device=DEV)).sum().item()     # eager work in between
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    got = [out_g] + [p.grad for p in params]
    for a, b in zip(want, got):
      assert torch.equal(a, b), (replay, kind)


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_column_sums(dtype):
  """The bias gradient's column sums on each of its three kernels (16-byte pieces, the flat run
  for few channels, one channel per lane) against an fp64 sum, and the same bits on a second run."""
  from ocnn_amd.nn.octree_conv import column_sum
  g = torch.Generator().manual_seed(3)
  for rows, C in [(1, 1), (7, 3), (1000, 4), (30011, 5), (4097, 7), (50000, 12), (2500, 40), (999, 100),
                  (70000, 64), (1234, 96), (300, 257), (513, 300), (100000, 8)]:
    say('column sums', dtype, rows, C)
    x = torch.randn(rows, C, generator=g).to(dtype).to(DEV)
    got = column_sum(x)
    want = x.double().sum(0)
    tol = 1e-5 if dtype == torch.float32 else 4e-3
    assert got.dtype == dtype and tuple(got.shape) == (C,)
    assert float((got.double() - want).abs().max()) <= tol * max(1.0, float(want.abs().max())) + tol * rows ** 0.5
    assert torch.equal(got, column_sum(x))


def test_the_documented_call_sequence_of_the_abi():
  """The calls a binder makes, in the order the integration notes give them, with nothing of the
  Python layer in between: tile plan by count / offsets / fill (six statistics, one read-back),
  the library's choice of the kernel, the register-resident gather on the plan, then the pair plan
  (slot counts, lists on the host, count, fill) and the pair-plan gather and weight gradient -
  against the plan-free entry points on the same table."""
  from ctypes import byref, c_int, c_int32, c_int64
  L = _lib.lib()
  g = torch.Generator().manual_seed(21)
  rows = rows_in = 128 * 300 + 17
  K, code, st = 27, _lib.DTYPE_CODE[torch.bfloat16], _lib.stream()
  table = _local_table(rows, rows_in, K, g, spread=30, empty=0.8).to(DEV)
  P = lambda t: t.data_ptr()
  say('abi sequence: tile plan')
  R = L.ocnn_tile_plan_rows()
  tiles = (rows + R - 1) // R
  ucount = torch.empty(tiles, dtype=torch.int32, device=DEV)
  tile_nnz = torch.empty(tiles, dtype=torch.int32, device=DEV)
  uptr = torch.empty(tiles + 1, dtype=torch.int32, device=DEV)
  stats = torch.empty(6, dtype=torch.int64, device=DEV)
  _lib.check(L.ocnn_tile_plan_count(P(table), rows, K, P(ucount), P(tile_nnz), st))
  _lib.check(L.ocnn_tile_plan_offsets(P(ucount), P(tile_nnz), tiles, 415, P(uptr), P(stats), st))
  over, dropped, total, umax, nnz, _ = stats.tolist()
  assert over == 0 and dropped == 0 and nnz == int((table >= 0).sum()) and 0 < umax <= 415
  urows = torch.empty(max(total, 1), dtype=torch.int32, device=DEV)
  loc = torch.empty((tiles, K, R), dtype=torch.int16, device=DEV)
  _lib.check(L.ocnn_tile_plan_fill(P(table), rows, K, P(uptr), P(urows), P(loc), st))
  occupancy, reuse = nnz / (rows * K), nnz / max(total, 1)

  def plain(x, w, cout):
    out = torch.empty(rows, cout, dtype=x.dtype, device=DEV)
    ws = torch.empty(L.ocnn_conv_gather_workspace_bytes(code, rows_in, K, x.shape[1], cout), dtype=torch.uint8, device=DEV)
    _lib.check(L.ocnn_conv_gather(code, P(x), rows_in, P(table), rows, K, P(w), x.shape[1], cout, 0, 0, None, P(out),
                                  P(ws), ws.numel(), st))
    return out

  say('abi sequence: 64 -> 64 on the plan')
  x = torch.randn(rows_in, 64, generator=g).to(torch.bfloat16).to(DEV)
  w = (torch.randn(K, 64, 64, generator=g) / 40).to(torch.bfloat16).to(DEV)
  assert L.ocnn_conv_gather_choose(code, rows_in, rows, K, 64, 64, 0, 1, umax, total, occupancy, reuse) == _lib.GATHER_RW
  ws = torch.empty(L.ocnn_conv_gather_workspace_bytes(code, rows_in, K, 64, 64), dtype=torch.uint8, device=DEV)
  out = torch.empty(rows, 64, dtype=torch.bfloat16, device=DEV)
  _lib.check(L.ocnn_conv_gather_rw(code, P(x), rows_in, P(loc), P(uptr), P(urows), umax, total, rows, K, P(w), 64, 64,
                                   0, 0, None, P(out), P(ws), ws.numel(), st))
  assert rel_err(out, f64(plain(x, w, 64))) < 1e-2

  say('abi sequence: pair plan, 96 -> 96')
  counts = torch.zeros(K, dtype=torch.int64, device=DEV)
  _lib.check(L.ocnn_pair_plan_slot_counts(P(loc), tiles, K, P(counts), st))
  h_counts = (c_int64 * K)(*counts.tolist())
  h_lists, h_list_count, h_bounds, n = (c_int32 * 32)(), (c_int64 * 32)(), (c_int32 * 5)(), c_int(0)
  _lib.check(L.ocnn_pair_plan_lists(K, h_counts, h_lists, h_list_count, h_bounds, byref(n)))
  nl = n.value
  lists = torch.tensor(list(h_lists)[:nl], dtype=torch.int32, device=DEV)
  nblk = torch.zeros(tiles * nl, dtype=torch.int32, device=DEV)
  _lib.check(L.ocnn_pair_plan_count(P(loc), tiles, K, P(lists), nl, P(nblk), st))
  cptr = torch.zeros(tiles * nl + 1, dtype=torch.int32, device=DEV)
  cptr[1:] = nblk.cumsum(0)
  n_blocks, max_blocks = int(cptr[-1]), int(nblk.view(tiles, nl).sum(1).max())
  ent = torch.empty(max(n_blocks, 1) * 16, dtype=torch.int32, device=DEV)
  _lib.check(L.ocnn_pair_plan_fill(P(loc), tiles, K, P(lists), nl, P(cptr), P(ent), st))
  x = torch.randn(rows_in, 96, generator=g).to(torch.bfloat16).to(DEV)
  w = (torch.randn(K, 96, 96, generator=g) / 50).to(torch.bfloat16).to(DEV)
  gr = torch.randn(rows, 96, generator=g).to(torch.bfloat16).to(DEV)
  assert L.ocnn_conv_gather_choose(code, rows_in, rows, K, 96, 96, 0, 1, umax, total, occupancy, reuse) == _lib.GATHER_SPARSE
  ws = torch.empty(L.ocnn_conv_gather_sparse_workspace_bytes(96, 96), dtype=torch.uint8, device=DEV)
  out = torch.empty(rows, 96, dtype=torch.bfloat16, device=DEV)
  _lib.check(L.ocnn_conv_gather_sparse(code, P(x), rows_in, P(uptr), P(urows), umax, total, P(cptr), P(ent), n_blocks,
                                       max_blocks, P(lists), nl, ctypes.addressof(h_bounds), rows, K, P(w), 96, 96, 0, 0,
                                       None, P(out), P(ws), ws.numel(), st))
  assert rel_err(out, f64(plain(x, w, 96))) < 1e-2
  ws2 = torch.empty(L.ocnn_conv_wgrad_sparse_workspace_bytes(rows, 96, 96), dtype=torch.uint8, device=DEV)
  gw = torch.empty(K, 96, 96, dtype=torch.bfloat16, device=DEV)
  _lib.check(L.ocnn_conv_wgrad_sparse(code, P(x), rows_in, 96, P(gr), rows, 96, P(uptr), P(urows), umax, total, P(cptr),
                                      P(ent), n_blocks, ctypes.addressof(h_lists), ctypes.addressof(h_list_count), nl, K, 1,
                                      P(gw), P(ws2), ws2.numel(), st))
  want = torch.empty(K, 96, 96, dtype=torch.bfloat16, device=DEV)
  ws3 = torch.empty(L.ocnn_conv_wgrad_workspace_bytes_for(code, rows_in, rows, K, 96, 96), dtype=torch.uint8, device=DEV)
  _lib.check(L.ocnn_conv_wgrad(code, P(x), rows_in, P(gr), P(table), rows, K, 96, 96, 0, P(want), P(ws3), ws3.numel(), st))
  assert rel_err(gw, f64(want)) < 1e-2
