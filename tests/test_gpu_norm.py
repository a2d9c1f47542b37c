"""GPU parity of the fused batch norm (+ ReLU) against torch.nn.BatchNorm1d + ReLU evaluated
in fp64 on the CPU: outputs, running statistics, all three gradients, training and evaluation
mode, every dtype."""

import os
import sys

import numpy as np
import pytest
from conftest import random_cases
import torch

from ocnn_amd.nn import BatchNormRelu1d

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = {torch.float32: 2e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def _ref(x, w, b, relu, training, rm, rv, momentum, eps, dy):
  """fp64 torch reference on the CPU; returns y, dx, dw, db and the updated running stats."""
  bn = torch.nn.BatchNorm1d(x.shape[1], eps=eps, momentum=momentum).double()
  with torch.no_grad():
    bn.weight.copy_(w.double()); bn.bias.copy_(b.double())
    bn.running_mean.copy_(rm.double()); bn.running_var.copy_(rv.double())
  bn.train(training)
  xd = x.double().requires_grad_()
  y = bn(xd)
  if relu:
    y = torch.relu(y)
  y.backward(dy.double())
  return y.detach(), xd.grad, bn.weight.grad, bn.bias.grad, bn.running_mean.clone(), bn.running_var.clone()


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('relu', [False, True])
@pytest.mark.parametrize('training', [True, False])
def test_batch_norm_relu_vs_torch(dtype, relu, training):
  g = torch.Generator().manual_seed(11)
  for rows, c in [(1000, 32), (4133, 96), (257, 8), (20000, 256), (3, 64)]:
    say('batch norm', dtype, relu, training, rows, c)
    x = (torch.randn(rows, c, generator=g) * 1.5 + 3.0).to(dtype)          # a mean well away from zero
    w = (torch.rand(c, generator=g) + 0.5).to(dtype).float()               # parameters the dtype holds exactly
    b = (torch.randn(c, generator=g) * 0.3).to(dtype).float()
    rm = (torch.randn(c, generator=g) * 0.1 + 3.0).to(dtype).float()
    rv = (torch.rand(c, generator=g) + 1.5).to(dtype).float()
    dy = torch.randn(rows, c, generator=g).to(dtype)
    want = _ref(x.float(), w, b, relu, training, rm, rv, 0.1, 1e-5, dy.float())
    bn = BatchNormRelu1d(c, relu=relu).to(DEV)
    with torch.no_grad():
      bn.weight.copy_(w); bn.bias.copy_(b); bn.running_mean.copy_(rm); bn.running_var.copy_(rv)
    bn = bn.to(dtype) if dtype != torch.float32 else bn
    bn.train(training)
    xg = x.to(DEV).requires_grad_()
    y = bn(xg)
    assert y.dtype == dtype
    y.backward(dy.to(DEV))
    tol = TOL[dtype]
    scale = lambda t: max(1.0, float(t.abs().max()))
    assert float((y.detach().double().cpu() - want[0]).abs().max()) <= tol * scale(want[0])
    # where the pre-activation is within rounding of zero the ReLU mask is a coin toss
    sure = torch.ones_like(want[0], dtype=torch.bool)
    if relu:
      mu = want[4] if not training else x.double().mean(0)
      sd = (want[5] + 1e-5).sqrt() if not training else (x.double().var(0, unbiased=False) + 1e-5).sqrt()
      z = (x.double() - (rm.double() if not training else mu)) / ((rv.double() + 1e-5).sqrt() if not training else sd) * w.double() + b.double()
      sure = z.abs() > 1e-3
    assert float(((xg.grad.double().cpu() - want[1]) * sure).abs().max()) <= 4 * tol * scale(want[1])
    assert int((~sure).sum()) < 0.01 * sure.numel()
    # parameter gradients are sums over the rows: relative to their size
    assert float((bn.weight.grad.double().cpu() - want[2]).abs().max()) <= 4 * tol * scale(want[2])
    assert float((bn.bias.grad.double().cpu() - want[3]).abs().max()) <= 4 * tol * scale(want[3])
    assert float((bn.running_mean.double().cpu() - want[4]).abs().max()) <= max(tol, 1e-3 if dtype != torch.float32 else 0) * scale(want[4])
    assert float((bn.running_var.double().cpu() - want[5]).abs().max()) <= max(tol, 1e-2 if dtype != torch.float32 else 0) * scale(want[5])
    assert int(bn.num_batches_tracked) == (1 if training else 0)
    # the same bits on a second run (fixed reduction order)
    bn.zero_grad()
    x2 = x.to(DEV).requires_grad_()
    y2 = bn(x2) if not training else None
    if y2 is not None:
      assert torch.equal(y2, y)


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('training', [True, False])
def test_batch_norm_residual_relu_vs_torch(dtype, training):
  """relu(bn(x) + residual) in one pass (the tail of a residual block) against torch's
  BatchNorm1d + add + ReLU in fp64: output, both input gradients, parameter gradients."""
  g = torch.Generator().manual_seed(13)
  for rows, c in [(1000, 32), (4133, 96), (20000, 256)]:
    say('batch norm + residual', dtype, training, rows, c)
    x = (torch.randn(rows, c, generator=g) * 1.5 + 1.0).to(dtype)
    res = torch.randn(rows, c, generator=g).to(dtype)
    dy = torch.randn(rows, c, generator=g).to(dtype)
    w = (torch.rand(c, generator=g) + 0.5).to(dtype).float()
    b = (torch.randn(c, generator=g) * 0.3).to(dtype).float()
    ref = torch.nn.BatchNorm1d(c).double()
    with torch.no_grad():
      ref.weight.copy_(w); ref.bias.copy_(b); ref.running_mean.fill_(1.0); ref.running_var.fill_(2.0)
    ref.train(training)
    xr, rr = x.double().requires_grad_(), res.double().requires_grad_()
    pre = ref(xr) + rr
    yr = torch.relu(pre)
    yr.backward(dy.double())
    bn = BatchNormRelu1d(c, relu=False).to(DEV)
    with torch.no_grad():
      bn.weight.copy_(w); bn.bias.copy_(b); bn.running_mean.fill_(1.0); bn.running_var.fill_(2.0)
    bn = bn.to(dtype) if dtype != torch.float32 else bn
    bn.train(training)
    xg, rg = x.to(DEV).requires_grad_(), res.to(DEV).requires_grad_()
    y = bn(xg, residual=rg, relu=True)
    y.backward(dy.to(DEV))
    tol = TOL[dtype]
    scale = lambda t: max(1.0, float(t.abs().max()))
    assert float((y.detach().double().cpu() - yr.detach()).abs().max()) <= 2 * tol * scale(yr)
    sure = pre.detach().abs() > 2e-2 * (1 if dtype != torch.float32 else 1e-3)     # away from the ReLU's kink
    assert int((~sure).sum()) < 0.05 * sure.numel()
    assert float(((xg.grad.double().cpu() - xr.grad) * sure).abs().max()) <= 4 * tol * scale(xr.grad)
    assert float(((rg.grad.double().cpu() - rr.grad) * sure).abs().max()) <= 4 * tol * scale(rr.grad)
    # (parameter gradients are sums over the rows: an element at the kink may fall either way)
    slack = ((~sure) * dy.double().abs()).sum(0)
    assert bool(((bn.bias.grad.double().cpu() - ref.bias.grad).abs() <= 8 * tol * scale(ref.bias.grad) + slack).all())
    assert bool(((bn.weight.grad.double().cpu() - ref.weight.grad).abs()
                 <= 8 * tol * scale(ref.weight.grad) + 5 * slack).all())
    # only the residual's gradient wanted: dx is still computed for it, x gets none
    x3 = x.to(DEV)
    r3 = res.to(DEV).requires_grad_()
    for p_ in bn.parameters():
      p_.requires_grad_(False)
    y3 = bn(x3, residual=r3, relu=True)
    y3.backward(dy.to(DEV))
    assert torch.equal(r3.grad, rg.grad) and torch.equal(y3, y) == (not training or True)


def test_batch_norm_fallbacks_and_state_dict():
  """3-D inputs and odd channel counts take torch's path; the state_dict is BatchNorm1d's."""
  bn = BatchNormRelu1d(6, relu=True).to(DEV)
  ref = torch.nn.BatchNorm1d(6).to(DEV)
  ref.load_state_dict(bn.state_dict())
  x = torch.randn(50, 6, device=DEV)
  assert torch.allclose(bn(x), torch.relu(ref(x)), atol=1e-6)
  bn2 = BatchNormRelu1d(16, relu=False).to(DEV)
  ref2 = torch.nn.BatchNorm1d(16).to(DEV)
  ref2.load_state_dict(bn2.state_dict())
  x = torch.randn(200, 16, device=DEV)
  assert torch.allclose(bn2(x), ref2(x), atol=1e-5)
  assert torch.allclose(bn2.running_var, ref2.running_var, atol=1e-6)
  x3 = torch.randn(4, 16, 10, device=DEV)
  assert torch.allclose(bn2(x3), ref2(x3), atol=1e-5)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
@pytest.mark.parametrize('cin,cout,bias', [(96, 64, False), (64, 16, True), (256, 128, False), (128, 512, True)])
def test_conv1x1_on_package_kernels(dtype, cin, cout, bias):
  """modules.Conv1x1 on many rows (the package's GEMM kernels) against torch.nn.Linear in fp64:
  output and all gradients."""
  from ocnn_amd import modules
  g = torch.Generator().manual_seed(cin + cout)
  rows = 5000
  m = modules.Conv1x1(cin, cout, use_bias=bias).to(DEV).to(dtype)
  x = torch.randn(rows, cin, generator=g).to(dtype)
  dy = torch.randn(rows, cout, generator=g).to(dtype)
  ref = torch.nn.Linear(cin, cout, bias).double()
  with torch.no_grad():
    ref.weight.copy_(m.linear.weight.double().cpu())
    if bias:
      ref.bias.copy_(m.linear.bias.double().cpu())
  xd = x.double().requires_grad_()
  ref(xd).backward(dy.double())
  xg = x.to(DEV).requires_grad_()
  y = m(xg)
  y.backward(dy.to(DEV))
  tol = 4e-3 if dtype == torch.float16 else 2e-2
  rel = lambda a, b: float((a.double().cpu() - b).abs().max() / b.abs().max())
  assert rel(y.detach(), ref(x.double()).detach()) < tol
  assert rel(xg.grad, xd.grad) < tol
  assert rel(m.linear.weight.grad, ref.weight.grad) < tol
  if bias:
    assert rel(m.linear.bias.grad, ref.bias.grad) < tol
  # few rows: torch's Linear
  small = torch.randn(10, cin, generator=g).to(dtype).to(DEV)
  assert torch.equal(m(small), m.linear(small))


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_conv1x1_narrow_head(dtype):
  """modules.Conv1x1 with few output channels on many rows (64 -> 10, a classification head):
  torch's GEMMs for output and input gradient, the package's split reduction for the weight
  gradient; against torch.nn.Linear in fp64, and the same bits on a second run."""
  from ocnn_amd import modules
  g = torch.Generator().manual_seed(7)
  rows, cin, cout = 70000, 64, 10
  m = modules.Conv1x1(cin, cout, use_bias=True).to(DEV).to(dtype)
  x = torch.randn(rows, cin, generator=g).to(dtype)
  dy = torch.randn(rows, cout, generator=g).to(dtype)
  ref = torch.nn.Linear(cin, cout, True).double()
  with torch.no_grad():
    ref.weight.copy_(m.linear.weight.double().cpu())
    ref.bias.copy_(m.linear.bias.double().cpu())
  xd = x.double().requires_grad_()
  ref(xd).backward(dy.double())
  grads = []
  for _ in range(2):
    m.zero_grad()
    xg = x.to(DEV).requires_grad_()
    y = m(xg)
    assert y.grad_fn is not None and 'RowsLinearNarrow' in type(y.grad_fn).__name__
    y.backward(dy.to(DEV))
    grads.append(m.linear.weight.grad.clone())
  tol = 4e-3 if dtype == torch.float16 else 2e-2
  rel = lambda a, b: float((a.double().cpu() - b).abs().max() / b.abs().max())
  assert rel(y.detach(), ref(x.double()).detach()) < tol
  assert rel(xg.grad, xd.grad) < tol
  assert rel(m.linear.weight.grad, ref.weight.grad) < tol
  assert rel(m.linear.bias.grad, ref.bias.grad) < tol
  assert torch.equal(grads[0], grads[1])


@pytest.mark.parametrize('cin,cout', [(32, 32), (32, 64)])
@pytest.mark.parametrize('nempty', [False, True])
def test_residual_block_is_its_parts(cin, cout, nempty):
  """modules.OctreeResBlock2 / OctreeResBlocks (ocnn/modules/resblocks.py:65-99, 134-159): the
  block with its fused tail (sum with the shortcut and ReLU inside the last batch norm's pass)
  against the same layers put together from torch.nn.BatchNorm1d, torch.nn.Linear and separate
  additions, fp32, training mode: output, input gradient, every parameter gradient and the
  running statistics."""
  import copy
  from ocnn_amd import modules, synthetic
  from ocnn_amd.nn import OctreeConv
  from ocnn_amd.octree import Octree, Points
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 2, 31, n=6000)
  o = Octree(5, 2, batch_size=2)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=2))
  o.construct_all_neigh()
  depth = 5
  rows = int(o.nnum_nempty[depth] if nempty else o.nnum[depth])
  torch.manual_seed(cin + cout)
  blk = modules.OctreeResBlocks(cin, cout, 2, bottleneck=1, nempty=nempty).to(DEV)
  for p in blk.parameters():
    if p.dim() == 1:
      p.data.uniform_(0.5, 1.5)
  say('residual blocks', cin, cout, 'nempty', nempty, 'rows', rows)

  class Parts(torch.nn.Module):
    """One block from library layers; the parameters are those of `b`."""
    def __init__(self, b):
      super().__init__()
      self.ca, self.cb = copy.deepcopy(b.conv3x3a.conv), copy.deepcopy(b.conv3x3b.conv)
      def bn_of(m):
        t = torch.nn.BatchNorm1d(m.num_features, m.eps, m.momentum).to(DEV)
        t.load_state_dict({k: v.clone() for k, v in m.state_dict().items()})
        return t
      self.ba, self.bb = bn_of(b.conv3x3a.bn), bn_of(b.conv3x3b.bn)
      self.proj = None
      if hasattr(b, 'conv1x1'):
        self.proj = copy.deepcopy(b.conv1x1.conv.linear)
        self.bp = bn_of(b.conv1x1.bn)
    def forward(self, x, octree, depth):
      y = torch.relu(self.ba(self.ca(x, octree, depth)))
      y = self.bb(self.cb(y, octree, depth))
      s = x if self.proj is None else self.bp(self.proj(x))
      return torch.relu(y + s)

  parts = torch.nn.ModuleList([Parts(b) for b in blk.resblks])
  x = torch.randn(rows, cin, device=DEV)
  dy = torch.randn(rows, cout, device=DEV)
  xa = x.clone().requires_grad_()
  ya = blk(xa, o, depth)
  ya.backward(dy)
  xb = x.clone().requires_grad_()
  yb = xb
  for p in parts:
    yb = p(yb, o, depth)
  yb.backward(dy)
  # (in the 2-norm: a pre-activation within rounding of zero may fall on either side of the
  # ReLU in the two forms, which moves single entries of the gradients by O(1))
  # (the gradients before a batch norm amplify this by 1 / sigma: 5e-3; a wiring error is O(1))
  close = lambda a, b: float((a.detach() - b.detach()).norm()) <= 5e-3 * float(b.detach().norm())
  assert close(ya, yb) and close(xa.grad, xb.grad)
  for b, p in zip(blk.resblks, parts):
    pairs = [(b.conv3x3a.conv.weights, p.ca.weights), (b.conv3x3b.conv.weights, p.cb.weights),
             (b.conv3x3a.bn.weight, p.ba.weight), (b.conv3x3a.bn.bias, p.ba.bias),
             (b.conv3x3b.bn.weight, p.bb.weight), (b.conv3x3b.bn.bias, p.bb.bias)]
    stats = [(b.conv3x3a.bn, p.ba), (b.conv3x3b.bn, p.bb)]
    if p.proj is not None:
      pairs += [(b.conv1x1.conv.linear.weight, p.proj.weight), (b.conv1x1.bn.weight, p.bp.weight),
                (b.conv1x1.bn.bias, p.bp.bias)]
      stats.append((b.conv1x1.bn, p.bp))
    for i, (u, v) in enumerate(pairs):
      assert close(u.grad, v.grad), (i, float((u.grad - v.grad).norm()), float(v.grad.norm()))
    for u, v in stats:
      assert close(u.running_mean, v.running_mean) and close(u.running_var, v.running_var)
      assert int(u.num_batches_tracked) == int(v.num_batches_tracked) == 1


def test_random_batch_norms_vs_torch():
  """Random shapes (2 .. 200 000 rows, 4 .. 2048 channels incl. counts that are no power of two),
  dtypes, training / evaluation, with and without ReLU and residual, against torch's batch norm in
  fp64: output, input gradient and both parameter gradients.  The reference takes the ReLU's mask
  from the output of the kernel (where the value before the ReLU is within rounding of zero the mask
  is a coin toss in any arithmetic), after checking that it differs from the fp64 mask nowhere
  else.  OCNN_TEST_CASES sets the number of cases (default 40)."""
  for case in random_cases(40):
    rng = np.random.default_rng(7000 + case)
    rows = int(rng.choice([2, 3, 63, 64, 65, 1000, 4097, 50000, 200000]))
    dtype = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    c = int(rng.choice([8, 16, 24, 40, 64, 96, 128, 200, 256, 512, 1024, 2048] +
                       ([4, 12, 36] if dtype == torch.float32 else [])))
    if rows * c > 3e7:
      rows = max(2, int(3e7) // c)
    relu, training = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    res = bool(rng.integers(0, 2)) and relu
    say('random batch norm', case, rows, c, dtype, 'relu', relu, 'training', training, 'residual', res)
    g = torch.Generator().manual_seed(case)
    x = (torch.randn(rows, c, generator=g) * 1.5 + 3.0).to(dtype)
    w = (torch.rand(c, generator=g) + 0.5).to(dtype).float()
    b = (torch.randn(c, generator=g) * 0.3).to(dtype).float()
    rm = (torch.randn(c, generator=g) * 0.1 + 3.0).to(dtype).float()
    rv = (torch.rand(c, generator=g) + 1.5).to(dtype).float()
    dy = torch.randn(rows, c, generator=g).to(dtype)
    r = torch.randn(rows, c, generator=g).to(dtype) if res else None
    bn64 = torch.nn.BatchNorm1d(c, eps=1e-5, momentum=0.1).double()
    with torch.no_grad():
      bn64.weight.copy_(w.double()); bn64.bias.copy_(b.double())
      bn64.running_mean.copy_(rm.double()); bn64.running_var.copy_(rv.double())
    bn64.train(training)
    xd = x.double().requires_grad_()
    pre = bn64(xd)
    if res:
      pre = pre + r.double()
    bn = BatchNormRelu1d(c, relu=relu).to(DEV)
    with torch.no_grad():
      bn.weight.copy_(w); bn.bias.copy_(b); bn.running_mean.copy_(rm); bn.running_var.copy_(rv)
    bn = bn.to(dtype) if dtype != torch.float32 else bn
    bn.train(training)
    xg = x.to(DEV).requires_grad_()
    y = bn(xg, r.to(DEV)) if res else bn(xg)
    y.backward(dy.to(DEV))
    mask = (y.detach().cpu() > 0).double() if relu else torch.ones_like(pre)
    if relu:
      near_zero = (4e-2 if dtype != torch.float32 else 1e-4) * (1 + (r.double().abs() if res else 0))
      assert not bool((((pre.detach() > 0).double() != mask) & (pre.detach().abs() > near_zero)).any()), case
    y64 = pre * mask
    y64.backward(dy.double())
    tol = TOL[dtype] * (8 if rows < 16 else 1)      # (statistics over a handful of rows are ill-conditioned in 16 bits)
    sc = lambda t: max(1.0, float(t.abs().max()))
    assert float((y.detach().double().cpu() - y64.detach()).abs().max()) <= (2 if res else 1) * tol * sc(y64.detach()), case
    assert float((xg.grad.double().cpu() - xd.grad).abs().max()) <= 6 * tol * sc(xd.grad), case
    assert float((bn.weight.grad.double().cpu() - bn64.weight.grad).abs().max()) <= 16 * tol * sc(bn64.weight.grad), case
    assert float((bn.bias.grad.double().cpu() - bn64.bias.grad).abs().max()) <= 6 * tol * sc(bn64.bias.grad), case
