"""GPU parity on the workloads the benchmark configurations name, each on its own octree.

  configs[0]  one sphere cloud of 20 000 points, depth 6, OctreeConv 3x3x3 32 -> 32 in fp32:
              the whole layer (out, data gradient, weight gradient) against the fp64 oracle,
              octree and neighbour table bit exact against the oracle
  configs[1]  batch 8 x 100 000 points, depth 8, 64 -> 64 in fp16 / bf16: every slot of the
              weight gradient and sampled rows of the output and of the data gradient against
              the fp64 definition (the adjoint scalars alone would let a few wrong rows pass)
  configs[2]  the same batch in bf16: OctreeConv 2x2x2 stride 2 64 -> 128 (depth 8 -> 7),
              OctreeDeconv 2x2x2 stride 2 128 -> 64 (depth 7 -> 8) and OctreeDWConv 3x3x3 on 128
              channels at depth 7, each through its module: every slot of the weight gradient,
              sampled rows of the output and of the data gradient against the fp64 definition,
              and the rows of the empty nodes of the padded tensors exactly zero
  configs[3]  batch 4 x 250 000 points (planes + spheres), depth 9: integer invariants of
              the build and the tables, then 32 -> 32 at depth 9 and 256 -> 256 at depth 6 in
              bf16 the same way

Tolerances: fp32 1e-4, 16-bit 2e-2 of the largest magnitude of the expected tensor (the bound
the task states); the sampled rows are also held row by row to the same fraction of the
row's own largest expected magnitude x 4 (a wrong row cannot hide behind a large one).

The full-size definitions are evaluated in fp64 with plain torch indexing and matmul on the
device (no kernel of this package): the data gradient in its scatter form, from the table
entries that point at a sampled row, so that it does not lean on the table's symmetry.
"""

import sys

import numpy as np
import pytest
import torch

from ocnn_amd import synthetic
from ocnn_amd.nn import OctreeConv, OctreeDeconv, OctreeDWConv
from ocnn_amd.octree import Octree, Points, xyz2key
from oracle import conv_ref as C
from oracle import octree_ref as R

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def f64(t):
  return t.detach().double().cpu().numpy()


def rel(got, want):
  """max |got - want| over the largest |want| (both torch, any device)."""
  want = want.double()
  return float((got.double() - want).abs().max() / want.abs().max().clamp_min(1e-30))


def rel_rows(got, want):
  """worst row: max |got - want| of the row over the row's own largest |want|."""
  want = want.double()
  scale = want.abs().amax(1).clamp_min(1e-30)
  return float(((got.double() - want).abs().amax(1) / scale).max())


def build(maker, batch, seed, n, depth):
  if batch == 1:
    pts, nrm = maker(n, seed=seed)
    bid = None
  else:
    pts, nrm, bid = synthetic.batch_clouds(maker, batch, seed, n=n)
  pc = Points(pts.to(DEV), nrm.to(DEV), batch_id=None if bid is None else bid.to(DEV), batch_size=batch)
  o = Octree(depth, 2, batch_size=batch)
  idx = o.build_octree(pc)
  o.construct_all_neigh()
  return o, idx, pts, nrm, bid


def integer_invariants(o, idx, pts, bid, depth):
  """What must hold of any octree and its tables, whatever the size."""
  assert int(idx.max()) + 1 == int(o.nnum_nempty[depth])
  for d in range(3, depth + 1):
    k = o.keys[d]
    assert bool((k[1:] > k[:-1]).all())                                 # sorted, unique
    assert int(o.nnum[d]) == 8 * int(o.nnum_nempty[d - 1])
    c = o.children[d]
    assert torch.equal(c[c >= 0].long(), torch.arange(int(o.nnum_nempty[d]), device=DEV))
    t = o._table(d, '333', 1, False).long()
    n = t.shape[0]
    assert torch.equal(t[:, 13], torch.arange(n, device=DEV))            # centre slot = itself
    rows, slots = torch.nonzero(t >= 0, as_tuple=True)
    assert torch.equal(t[t[rows, slots], 26 - slots], rows)              # central symmetry
    del rows, slots, t
    assert torch.equal(o.keys[d] >> 3 & ((1 << 45) - 1),
                       (o.keys[d - 1][o.nempty_index(d - 1)] & ((1 << 48) - 1)).repeat_interleave(8))
    t2 = o._table(d, '222', 2, False).long()
    assert torch.equal(t2, (torch.arange(n // 8, device=DEV) * 8).unsqueeze(1) + torch.arange(8, device=DEV))
  leaf_key = o.keys[depth][o.nempty_index(depth)]
  p = (pts.to(DEV) + 1.0) * float(2 ** (depth - 1))
  b = None if bid is None else bid.to(DEV).view(-1)
  assert torch.equal(leaf_key[idx], xyz2key(p[:, 0], p[:, 1], p[:, 2], b, depth))


def definition_checks(o, depth, ch, dtype, nempty, seed):
  """One OctreeConv 3x3x3 ch -> ch forward + backward through the module; every slot of the
  weight gradient, every row of the output and of the data gradient against fp64 (a row's error
  over its own largest expected magnitude, or over a twentieth of the tensor's if that is larger)."""
  g = torch.Generator().manual_seed(seed)
  t = o._table(depth, '333', 1, nempty)
  rows = t.shape[0]
  conv = OctreeConv(ch, ch, [3], 1, nempty=nempty)
  with torch.no_grad():
    conv.weights.copy_(torch.randn(conv.weights.shape, generator=g) / (27 * ch) ** 0.5)
  conv = conv.to(DEV).to(dtype)
  x = torch.randn(rows, ch, generator=g).to(dtype).to(DEV).requires_grad_()
  gout = torch.randn(rows, ch, generator=g).to(dtype).to(DEV)
  out = conv(x, o, depth)
  out.backward(gout)
  assert out.dtype == dtype and x.grad.dtype == dtype and conv.weights.grad.dtype == dtype
  W = conv.weights.detach().double()
  xd = x.detach()
  tol = TOL[dtype]

  # every slot of the weight gradient: gW[k] = sum_i [t_ik >= 0] x[t_ik]^T (x) g[i]
  want_w = torch.empty(27, ch, ch, dtype=torch.float64, device=DEV)
  for k in range(27):
    v = torch.nonzero(t[:, k] >= 0).squeeze(1)
    want_w[k] = xd[t[v, k].long()].double().T @ gout[v].double()
  err_w = rel(conv.weights.grad, want_w)
  err_w_slot = max(rel(conv.weights.grad[k], want_w[k]) for k in range(27))

  # EVERY row of the output: out[i] = sum_k [t_ik >= 0] x[t_ik] @ W[k] (in pieces of 2^18 rows)
  err_o = err_o_row = 0.0
  scale_o = None
  piece = 1 << 18
  want_all = []
  for r0 in range(0, rows, piece):
    ts = t[r0:r0 + piece].long()
    want_o = torch.zeros(ts.shape[0], ch, dtype=torch.float64, device=DEV)
    for k in range(27):
      v = ts[:, k] >= 0
      want_o[v] += xd[ts[v, k]].double() @ W[k]
    want_all.append(want_o)
  scale_o = max(float(w.abs().max()) for w in want_all)
  for r0, want_o in zip(range(0, rows, piece), want_all):
    d = (out[r0:r0 + piece].detach().double() - want_o).abs()
    err_o = max(err_o, float(d.max()) / scale_o)
    err_o_row = max(err_o_row, float((d.amax(1) / want_o.abs().amax(1).clamp_min(0.05 * scale_o)).max()))
  del want_all

  # EVERY row of the data gradient, scatter form: gin[j] = sum over the entries (i, k) of the
  # table that hold j of g[i] @ W[k]^T
  want_g = torch.zeros(rows, ch, dtype=torch.float64, device=DEV)
  for k in range(27):
    tk = t[:, k].long()
    i = torch.nonzero(tk >= 0).squeeze(1)
    want_g.index_add_(0, tk[i], gout[i].double() @ W[k].T)
  d = (x.grad.double() - want_g).abs()
  scale_g = float(want_g.abs().max())
  err_g = float(d.max()) / scale_g
  err_g_row = float((d.amax(1) / want_g.abs().amax(1).clamp_min(0.05 * scale_g)).max())
  del want_g, d
  say('   rows %d  nnz/row %.2f  rel err: gW %.2e (worst slot %.2e)  out %.2e (worst row %.2e)  '
      'gdata %.2e (worst row %.2e)' % (rows, float((t >= 0).sum()) / rows, err_w, err_w_slot, err_o,
                                       err_o_row, err_g, err_g_row))
  assert err_w < tol and err_w_slot < tol
  assert err_o < tol and err_o_row < 4 * tol
  assert err_g < tol and err_g_row < 4 * tol


def table_definition_checks(t, fine, coarse, fwd, bwd, outer, got_gather, got_scatter, got_w, dtype, g):
  """The three passes of a layer over the table t (rows, K), whose entries index the rows of
  `fine`, against their fp64 definitions:
    gather   rows i:  sum_k [t_ik >= 0] fwd(k, fine[t_ik])            (every row of got_gather)
    scatter  rows j:  sum over the entries (i, k) that hold j of bwd(k, coarse[i])
                                                                    (every row of got_scatter)  
    weights  slot k:  outer(fine[t_ik], coarse[i]) over the rows with t_ik >= 0   (all of got_w)
  """
  rows, K = t.shape
  tol = TOL[dtype]
  want_w = []
  for k in range(K):
    v = torch.nonzero(t[:, k] >= 0).squeeze(1)
    want_w.append(outer(fine[t[v, k].long()].double(), coarse[v].double()))
  want_w = torch.stack(want_w)
  err_w = rel(got_w.reshape(want_w.shape), want_w)
  err_w_slot = max(rel(got_w.reshape(want_w.shape)[k], want_w[k]) for k in range(K))

  def row_errors(got, want):
    d = (got.detach().double() - want).abs()
    scale = float(want.abs().max())
    return float(d.max()) / scale, float((d.amax(1) / want.abs().amax(1).clamp_min(0.05 * scale)).max())

  # every row of the gather, in pieces of 2^18 rows
  err_o = err_o_row = 0.0
  wants = []
  for r0 in range(0, rows, 1 << 18):
    ts = t[r0:r0 + (1 << 18)].long()
    want_o = None
    for k in range(K):
      v = ts[:, k] >= 0
      term = fwd(k, fine[ts[:, k].clamp_min(0)].double()) * v.unsqueeze(1)
      want_o = term if want_o is None else want_o + term
    wants.append(want_o)
  err_o, err_o_row = row_errors(got_gather, torch.cat(wants))
  del wants

  # every row of the scatter
  n_fine = fine.shape[0]
  want_g = torch.zeros(n_fine, got_scatter.shape[1], dtype=torch.float64, device=DEV)
  for k in range(K):
    tk = t[:, k].long()
    i = torch.nonzero(tk >= 0).squeeze(1)
    want_g.index_add_(0, tk[i], bwd(k, coarse[i].double()))
  err_g, err_g_row = row_errors(got_scatter, want_g)
  del want_g
  say('   table %d x %d, %.2f entries a row: rel err weights %.2e (worst slot %.2e)  gather %.2e (worst row %.2e)  '
      'scatter %.2e (worst row %.2e)' % (rows, K, float((t >= 0).sum()) / rows, err_w, err_w_slot, err_o,
                                         err_o_row, err_g, err_g_row))
  assert err_w < tol and err_w_slot < tol
  assert err_o < tol and err_o_row < 4 * tol
  assert err_g < tol and err_g_row < 4 * tol


# ---------------------------------------------------------------------------------------------

def test_config2_stride2_conv_deconv_and_depthwise_bf16():
  dtype = torch.bfloat16
  say('configs[2]: 8 x 100 000 points, depth 8, bf16')
  o, _, _, _, _ = build(synthetic.mixed_cloud, 8, 1001, 100000, 8)
  g = torch.Generator().manual_seed(41)
  n8, n7, p7 = int(o.nnum[8]), int(o.nnum[7]), int(o.nnum_nempty[7])
  assert n8 == 8 * p7
  t = o._table(8, '222', 2, False)                          # (non-empty nodes of depth 7, 8) -> rows of depth 8
  node7 = o.nempty_index(7)                                 # their rows among all nodes of depth 7
  empty7 = o.children[7] < 0

  say('  OctreeConv 2x2x2 stride 2, 64 -> 128, depth 8 -> 7')
  conv = OctreeConv(64, 128, [2], 2)
  with torch.no_grad():
    conv.weights.copy_(torch.randn(conv.weights.shape, generator=g) / (8 * 64) ** 0.5)
  conv = conv.to(DEV).to(dtype)
  x = torch.randn(n8, 64, generator=g).to(dtype).to(DEV).requires_grad_()
  gout = torch.randn(n7, 128, generator=g).to(dtype).to(DEV)      # (the rows of the empty nodes must not count)
  out = conv(x, o, 8)
  out.backward(gout)
  assert out.shape == (n7, 128) and out.dtype == dtype
  assert not bool(out[empty7].any())                        # octree_pad: zeros for the empty nodes
  W = conv.weights.detach().double()
  table_definition_checks(t, x.detach(), gout[node7], lambda k, r: r @ W[k], lambda k, r: r @ W[k].T,
                          lambda a, b: a.T @ b, out[node7], x.grad, conv.weights.grad, dtype, g)

  say('  OctreeDeconv 2x2x2 stride 2, 128 -> 64, depth 7 -> 8')
  deconv = OctreeDeconv(128, 64, [2], 2)
  with torch.no_grad():
    deconv.weights.copy_(torch.randn(deconv.weights.shape, generator=g) / (8 * 128) ** 0.5)
  deconv = deconv.to(DEV).to(dtype)
  x = torch.randn(n7, 128, generator=g).to(dtype).to(DEV).requires_grad_()   # a row for every node of depth 7
  gout = torch.randn(n8, 64, generator=g).to(dtype).to(DEV)
  out = deconv(x, o, 7)
  out.backward(gout)
  assert out.shape == (n8, 64) and x.grad.shape == (n7, 128)
  assert not bool(x.grad[empty7].any())                     # the rows the depad dropped get no gradient
  W = deconv.weights.detach().double()                      # (8, 64, 128)
  table_definition_checks(t, gout, x.detach()[node7], lambda k, r: r @ W[k], lambda k, r: r @ W[k].T,
                          lambda a, b: a.T @ b, x.grad[node7], out, deconv.weights.grad, dtype, g)

  say('  OctreeDWConv 3x3x3, 128 channels, depth 7')
  dw = OctreeDWConv(128, [3], 1)
  with torch.no_grad():
    dw.weights.copy_(torch.randn(dw.weights.shape, generator=g) / 27 ** 0.5)
  dw = dw.to(DEV).to(dtype)
  t7 = o._table(7, '333', 1, False)
  x = torch.randn(n7, 128, generator=g).to(dtype).to(DEV).requires_grad_()
  gout = torch.randn(n7, 128, generator=g).to(dtype).to(DEV)
  out = dw(x, o, 7)
  out.backward(gout)
  w = dw.weights.detach().double().view(27, 128)
  table_definition_checks(t7, x.detach(), gout, lambda k, r: r * w[k], lambda k, r: r * w[k],
                          lambda a, b: (a * b).sum(0), out, x.grad, dw.weights.grad, dtype, g)


@pytest.mark.parametrize('nempty', [False, True])
def test_config0_sphere_depth6_fp32(nempty):
  say('configs[0]: 20 000 points on a sphere, depth 6, 32 -> 32 fp32, nempty', nempty)
  o, idx, pts, nrm, _ = build(synthetic.sphere_cloud, 1, 1000, 20000, 6)
  ref, ref_idx = R.build_octree(pts.numpy(), nrm.numpy(), depth=6, full_depth=2)
  R.construct_all_neigh(ref)
  assert np.array_equal(torch.cat(o.keys).cpu().numpy(), np.concatenate(ref.keys))
  assert np.array_equal(torch.cat(o.children).cpu().numpy(), np.concatenate(ref.children))
  assert np.array_equal(idx.cpu().numpy(), ref_idx)
  for d in range(1, 7):
    assert np.array_equal(o.neighs[d].cpu().numpy(), ref.neighs[d]), d
  g = torch.Generator().manual_seed(1000)
  conv = OctreeConv(32, 32, [3], 1, nempty=nempty)
  with torch.no_grad():
    bound = 1.0 / (27 * 32) ** 0.5                       # the configuration's Kaiming-uniform bound
    conv.weights.copy_((torch.rand(conv.weights.shape, generator=g) * 2 - 1) * bound)
  conv = conv.to(DEV)
  rows = int(ref.nnum_nempty[6] if nempty else ref.nnum[6])
  data = torch.randn(rows, 32, generator=g)
  gout = torch.randn(rows, 32, generator=g)
  x = data.to(DEV).requires_grad_()
  out = conv(x, o, 6)
  out.backward(gout.to(DEV))
  want = C.conv_layer(ref, f64(data), f64(conv.weights), 6, [3], 1, nempty, grad=f64(gout))
  for name, got, exp in (('out', out, want[0]), ('gdata', x.grad, want[1]), ('gW', conv.weights.grad, want[2])):
    exp = torch.from_numpy(exp)
    e, er = rel(got.cpu(), exp), (rel_rows(got.cpu(), exp) if name != 'gW' else 0.0)
    say('   %-5s rel err %.2e  worst row %.2e' % (name, e, er))
    assert e < 1e-4 and er < 4e-4, name


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_config1_full_weight_gradient_and_sampled_rows(dtype):
  say('configs[1]: 8 x 100 000 points, depth 8, 64 -> 64', dtype)
  o, _, _, _, _ = build(synthetic.mixed_cloud, 8, 1001, 100000, 8)
  definition_checks(o, 8, 64, dtype, False, 31)
  say('configs[1], non-empty nodes only (the mode of the reference\'s published table)')
  definition_checks(o, 8, 64, dtype, True, 32)


def test_config3_depth9_build_and_layers():
  say('configs[3]: 4 x 250 000 points on planes and spheres, depth 9: build and tables')
  o, idx, pts, _, bid = build(synthetic.planes_cloud, 4, 1003, 250000, 9)
  say('   nnum', o.nnum.tolist(), 'nnum_nempty', o.nnum_nempty.tolist())
  integer_invariants(o, idx, pts, bid, 9)
  say('configs[3]: 32 -> 32 at depth 9, bf16')
  definition_checks(o, 9, 32, torch.bfloat16, False, 33)
  say('configs[3]: 256 -> 256 at depth 6, bf16')
  definition_checks(o, 6, 256, torch.bfloat16, False, 34)
  say('configs[3]: the same layers on non-empty nodes')
  definition_checks(o, 9, 32, torch.bfloat16, True, 35)
  definition_checks(o, 6, 256, torch.bfloat16, True, 36)


def test_layers_give_the_same_bits_on_every_run():
  """No kernel of the path sums in an order that depends on timing, and none may read a row
  before its load has landed: every layer shape of the benchmark configurations and of the
  kernel-shape x stride grid, at full size (8 x 100 000 points, depth 8), run four times on the
  same inputs - output, data gradient and weight gradient are the same bits every time.  (A
  wait that comes too early shows as a few differing rows in some runs; the oracle tests on
  small octrees, whose tiles are few, may never see it.)"""
  say('same bits on every run: 8 x 100 000 points, depth 8, bf16')
  o, _, _, _, _ = build(synthetic.mixed_cloud, 8, 1001, 100000, 8)
  rows = {(d, ne): int((o.nnum_nempty if ne else o.nnum)[d]) for d in (6, 7, 8) for ne in (False, True)}
  layers = [('conv', ks, 1, ne, ch, ch, 8) for ks in ([3], [3, 1, 1], [1, 3, 1], [3, 3, 1], [2])
            for ne in (False, True) for ch in (32, 64)]
  layers += [(kind, ks, 2, ne, 64, 64, 8 if kind == 'conv' else 7) for kind in ('conv', 'deconv')
             for ks in ([3], [3, 1, 1], [3, 3, 1], [2]) for ne in (False, True)]
  layers += [('conv', [2], 2, False, 64, 128, 8), ('deconv', [2], 2, False, 128, 64, 7), ('dwconv', [3], 1, False, 128, 128, 7),
             ('dwconv', [3], 1, True, 64, 64, 8), ('conv', [3], 1, True, 96, 96, 8), ('conv', [3], 1, True, 128, 96, 8),
             ('conv', [3], 1, True, 128, 128, 7), ('conv', [3], 1, False, 256, 256, 6), ('conv', [2], 2, True, 96, 96, 8),
             ('deconv', [2], 2, True, 96, 96, 7)]
  g = torch.Generator().manual_seed(77)
  for kind, ks, stride, ne, cin, cout, depth in layers:
    if kind == 'dwconv':
      mod = OctreeDWConv(cin, ks, stride, ne)
    else:
      mod = (OctreeConv if kind == 'conv' else OctreeDeconv)(cin, cout, ks, stride, ne)
    mod = mod.to(DEV).to(torch.bfloat16)
    n_in = rows[(depth, ne)]
    x = torch.randn(n_in, cin, generator=g).bfloat16().to(DEV).requires_grad_()
    first = None
    for run in range(4):
      x.grad = None
      mod.weights.grad = None
      out = mod(x, o, depth)
      if first is None:
        gout = torch.randn(out.shape, generator=g).bfloat16().to(DEV)
      out.backward(gout)
      now = (out.detach().clone(), x.grad.clone(), mod.weights.grad.clone())
      if first is None:
        first = now
        continue
      for name, a, b in zip(('output', 'data gradient', 'weight gradient'), first, now):
        if not torch.equal(a, b):
          d = (a.float() - b.float()).abs().view(a.shape[0], -1).amax(1)
          bad = d.nonzero().view(-1)
          raise AssertionError('%s of %s %s stride %d nempty %s %d -> %d differs in run %d: %d rows, first %s' % (
              name, kind, ks, stride, ne, cin, cout, run, bad.numel(), bad[:8].tolist()))
    say('   %s %s stride %d nempty %s %d -> %d depth %d: %d rows in, same bits 4 times' % (kind, ks, stride, ne, cin, cout, depth, n_in))


def test_the_ops_around_the_convolutions_on_more_than_2_31_elements():
  """Batch norm + ReLU (training mode, forward and backward), pad / depad, max pooling and the
  depth-wise convolution on the deepest layer of an octree of 8 x 1.1 M points at depth 11:
  49.9 M nodes x 64 channels = 3.2 G elements per tensor, where a 32-bit element index wraps.
  Against fp64 torch on the first, the last and random rows (and the rows around element
  2^31 and 2^32)."""
  from ocnn_amd.nn import BatchNormRelu1d, octree_pad, octree_depad, octree_max_pool
  say('ops on tensors of more than 2^31 elements')
  o, _, _, _, _ = build(synthetic.mixed_cloud, 8, 77, 1100000, 11)
  d, C = 11, 64
  n_all, n_ne = int(o.nnum[d]), int(o.nnum_nempty[d])
  assert n_all * C > 1 << 31
  g = torch.Generator(device=DEV).manual_seed(1)
  piece = 1 << 22
  sel = torch.cat([torch.arange(0, 1000, device=DEV), torch.arange(n_all - 1000, n_all, device=DEV),
                   torch.arange((1 << 31) // C - 500, (1 << 31) // C + 500, device=DEV),
                   torch.arange((1 << 32) // C - 500, (1 << 32) // C + 500, device=DEV).clamp_(max=n_all - 1),
                   torch.randint(0, n_all, (5000,), device=DEV, generator=g)])

  def close(got, want, tol=2e-2):
    err = float((got.double() - want).abs().max() / want.abs().max())
    assert err < tol, err
    return err

  # ---- batch norm + ReLU ----
  x = torch.randn(n_all, C, device=DEV, generator=g).bfloat16().requires_grad_()
  gy = torch.randn(n_all, C, device=DEV, generator=g).bfloat16()
  bn = BatchNormRelu1d(C, relu=True).to(DEV).bfloat16()
  with torch.no_grad():
    bn.weight.copy_(torch.rand(C, device=DEV, generator=g) + 0.5)
    bn.bias.copy_(torch.randn(C, device=DEV, generator=g) * 0.1)
  y = bn(x)
  y.backward(gy)
  xd = x.detach()
  mean = torch.zeros(C, device=DEV, dtype=torch.float64)
  sq = torch.zeros(C, device=DEV, dtype=torch.float64)
  for r0 in range(0, n_all, piece):
    xx = xd[r0:r0 + piece].double()
    mean += xx.sum(0)
    sq += (xx * xx).sum(0)
  mean /= n_all
  inv = 1.0 / torch.sqrt(sq / n_all - mean * mean + bn.eps)
  scale = bn.weight.detach().double() * inv
  shift = bn.bias.detach().double() - mean * scale
  e_fwd = close(y.detach()[sel], torch.relu(xd[sel].double() * scale + shift))
  s1 = torch.zeros(C, device=DEV, dtype=torch.float64)
  s2 = torch.zeros(C, device=DEV, dtype=torch.float64)
  for r0 in range(0, n_all, piece):
    xx = xd[r0:r0 + piece].double()
    gg = gy[r0:r0 + piece].double() * ((xx * scale + shift) > 0)
    s1 += gg.sum(0)
    s2 += (gg * (xx - mean) * inv).sum(0)
  xx = xd[sel].double()
  gg = gy[sel].double() * ((xx * scale + shift) > 0)
  e_bwd = close(x.grad[sel], scale * (gg - s1 / n_all - (xx - mean) * inv * s2 / n_all))
  close(bn.weight.grad, s2)
  close(bn.bias.grad, s1)
  say('   batch norm + ReLU, %d x %d: forward %.1e, backward %.1e' % (n_all, C, e_fwd, e_bwd))
  del x, y, gy, bn, xd
  torch.cuda.empty_cache()

  # ---- pad / depad, max pooling ----
  xn = torch.randn(n_ne, C, device=DEV, generator=g).bfloat16()
  p = octree_pad(xn, o, d)
  assert p.shape[0] == n_all and torch.equal(p[o.nempty_index(d)], xn) and torch.equal(octree_depad(p, o, d), xn)
  assert int(torch.count_nonzero(p)) == int(torch.count_nonzero(xn))                               # zeros elsewhere
  del p, xn
  xa = torch.randn(n_all, C, device=DEV, generator=g).bfloat16()
  pooled = octree_max_pool(xa, o, d, nempty=False)
  assert torch.equal(octree_depad(pooled, o, d - 1), xa.view(-1, 8, C).max(1).values)
  del xa, pooled
  torch.cuda.empty_cache()

  # ---- depth-wise convolution on the non-empty nodes ----
  dw = OctreeDWConv(C, [3], 1, nempty=True).to(DEV).bfloat16()
  xd = torch.randn(n_ne, C, device=DEV, generator=g).bfloat16()
  out = dw(xd, o, d)
  t = o._table(d, '333', 1, True)
  rows = torch.cat([torch.arange(0, 1000, device=DEV), torch.arange(n_ne - 1000, n_ne, device=DEV),
                    torch.randint(0, n_ne, (3000,), device=DEV, generator=g)])
  ts = t[rows].long()
  w = dw.weights.detach().double().view(27, C)
  want = torch.zeros(rows.numel(), C, dtype=torch.float64, device=DEV)
  for k in range(27):
    v = ts[:, k] >= 0
    want[v] += xd[ts[v, k]].double() * w[k]
  say('   depth-wise convolution on %d rows: %.1e' % (n_ne, close(out.detach()[rows], want)))

