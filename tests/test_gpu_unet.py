"""The assembled segmentation U-Net (ocnn_amd.unet.UNet, configs[4]) on the GPU.

Small octree, fp32: logits, loss and the gradient of EVERY parameter against a composition,
in fp64 on the CPU, of the oracle's layers (conv / deconv definitions, trilinear
interpolation) with torch's batch norm, ReLU and linear — the same parameters, same inputs.
Full size (8 x 150 000 points of indoor-like scenes, depth 9): the first block's output on all
rows against its fp64 definition in fp32 and bf16; then one forward + backward in bf16: loss and
all gradients finite, loss equal to the fp32 run of the same net within 16-bit rounding,
gradients pointing the same way as the fp32 ones.
"""

import sys

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from ocnn_amd import synthetic
from ocnn_amd.octree import Octree, Points
from ocnn_amd.unet import UNet, ENCODER_BLOCKS, DECODER_BLOCKS
from oracle import conv_ref as C
from oracle import interp_ref as I
from oracle import octree_ref as R

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


class _OracleLayer(torch.autograd.Function):
  """An oracle conv / deconv layer (numpy fp64) as an autograd node."""

  @staticmethod
  def forward(ctx, x, w, layer, oct, depth, ks, stride, nempty):
    ctx.args = (layer, oct, depth, ks, stride, nempty)
    ctx.save_for_backward(x, w)
    return torch.from_numpy(layer(oct, x.numpy(), w.numpy(), depth, ks, stride, nempty))

  @staticmethod
  def backward(ctx, grad):
    layer, oct, depth, ks, stride, nempty = ctx.args
    x, w = ctx.saved_tensors
    res = layer(oct, x.numpy(), w.numpy(), depth, ks, stride, nempty, grad=grad.contiguous().numpy())
    return (torch.from_numpy(res[1]), torch.from_numpy(res[2])) + (None,) * 6


class _OracleInterp(torch.autograd.Function):
  @staticmethod
  def forward(ctx, x, oct, depth, pts, nempty):
    ctx.args = (oct, depth, pts, nempty, x.shape[0])
    return torch.from_numpy(I.linear_pts(oct, x.numpy(), depth, pts, nempty)).to(x.dtype)

  @staticmethod
  def backward(ctx, grad):
    oct, depth, pts, nempty, rows = ctx.args
    return (torch.from_numpy(I.linear_pts_grad(oct, grad.numpy(), depth, pts, rows, nempty)).to(grad.dtype),) + (None,) * 4


class OracleUNet:
  """The network of ocnn/models/unet.py:16-105 over the oracle's layers; parameters by the
  names of the module tree (a state_dict of the GPU net, as fp64 leaves)."""

  def __init__(self, params, oct, nempty, running=None):
    self.p, self.oct, self.nempty, self.running = params, oct, nempty, running

  def bn(self, x, name):
    if self.running is not None:           # evaluation mode: the stored statistics
      mean, var = self.running[name + '.running_mean'], self.running[name + '.running_var']
      return F.batch_norm(x, mean.to(x.dtype), var.to(x.dtype), self.p[name + '.weight'], self.p[name + '.bias'],
                          False, 0.1, 1e-5)
    return F.batch_norm(x, None, None, self.p[name + '.weight'], self.p[name + '.bias'], True, 0.1, 1e-5)

  def conv(self, x, name, depth, ks=(3,), stride=1, deconv=False):
    layer = C.deconv_layer if deconv else C.conv_layer
    return _OracleLayer.apply(x, self.p[name + '.weights'], layer, self.oct, depth, ks, stride, self.nempty)

  def conv_bn_relu(self, x, name, depth, ks=(3,), stride=1, deconv=False):
    sub = 'deconv' if deconv else 'conv'
    return torch.relu(self.bn(self.conv(x, name + '.' + sub, depth, ks, stride, deconv), name + '.bn'))

  def resblock(self, x, name, depth):
    y = self.conv_bn_relu(x, name + '.conv3x3a', depth)
    y = self.bn(self.conv(y, name + '.conv3x3b.conv', depth), name + '.conv3x3b.bn')
    if name + '.conv1x1.conv.linear.weight' in self.p:
      x = self.bn(F.linear(x, self.p[name + '.conv1x1.conv.linear.weight']), name + '.conv1x1.bn')
    return torch.relu(y + x)

  def blocks(self, x, name, n, depth):
    for j in range(n):
      x = self.resblock(x, '%s.resblks.%d' % (name, j), depth)
    return x

  def __call__(self, data, depth, pts_octree_coords):
    feats = {depth: self.conv_bn_relu(data, 'conv1', depth)}
    for i, n in enumerate(ENCODER_BLOCKS):
      d = depth - i
      y = self.conv_bn_relu(feats[d], 'downsample.%d' % i, d, (2,), 2)
      feats[d - 1] = self.blocks(y, 'encoder.%d' % i, n, d - 1)
    d0 = depth - len(ENCODER_BLOCKS)
    x = feats[d0]
    for i, n in enumerate(DECODER_BLOCKS):
      d = d0 + i
      up = self.conv_bn_relu(x, 'upsample.%d' % i, d, (2,), 2, deconv=True)
      x = self.blocks(torch.cat([feats[d + 1], up], 1), 'decoder.%d' % i, n, d + 1)
    f = _OracleInterp.apply(x, self.oct, depth, pts_octree_coords, self.nempty)
    h = torch.relu(self.bn(F.linear(f, self.p['header.0.conv.linear.weight']), 'header.0.bn'))
    return F.linear(h, self.p['header.1.linear.weight'], self.p['header.1.linear.bias'])


def _loss(logits, labels):
  return F.cross_entropy(logits, labels)


@pytest.mark.parametrize('training', [False, True])
@pytest.mark.parametrize('nempty', [True, False])
def test_unet_small_fp32_against_oracle_layers(nempty, training):
  """training=False: batch norm with stored (random) statistics, a plain affine map per channel;
  the net is then well conditioned and every gradient must agree closely.  training=True: batch
  statistics; the coarse levels hold 16 .. 128 rows, the gradient of a layer in front of a batch
  norm is what is left after its mean and its projection on the output are taken out, and 36 of
  them sit between the first layer and the loss: on this net torch's own fp32 CPU arithmetic
  differs from fp64 by up to 5e-3 in single gradients (max norm), and the fp32 convolutions
  here carry 4e-6 per product (three bf16 MFMA passes), so those gradients are held loosely,
  logits and loss tightly in both modes."""
  depth, batch, n = 6, 2, 6000
  say('U-Net, fp32, depth 6, 2 x 6000 points, nempty', nempty, 'batch statistics' if training else
      'stored statistics', 'against oracle layers + torch fp64 batch norm')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, batch, 77, n=n)
  o = Octree(depth, 2, batch_size=batch)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=batch))
  o.construct_all_neigh()
  ref, _ = R.build_octree(pts.numpy(), nrm.numpy(), batch_id=bid.numpy(), depth=depth, full_depth=2,
                          batch_size=batch)
  R.construct_all_neigh(ref)
  feat = o.get_input_feature('ND', nempty)
  assert np.allclose(feat.cpu().numpy(), ref.get_input_feature('ND', nempty), atol=1e-6)
  query = torch.cat([pts, bid.float().view(-1, 1)], 1)
  labels = torch.randint(0, 10, (query.shape[0],), generator=torch.Generator().manual_seed(5))

  torch.manual_seed(3)
  net = UNet(feat.shape[1], 10, 'linear', nempty)
  with torch.no_grad():                       # batch-norm parameters and statistics away from 1 / 0
    g = torch.Generator().manual_seed(4)
    for name, p in net.named_parameters():
      if name.endswith('bn.weight'):
        p.copy_(0.5 + torch.rand(p.shape, generator=g))
      elif name.endswith('bn.bias'):
        p.copy_(0.2 * torch.randn(p.shape, generator=g))
    for name, b in net.named_buffers():
      if name.endswith('running_mean'):
        b.copy_(0.1 * torch.randn(b.shape, generator=g))
      elif name.endswith('running_var'):
        b.copy_(0.5 + torch.rand(b.shape, generator=g))
  net = net.to(DEV).train(training)
  running = None if training else {k: v.detach().double().cpu() for k, v in net.named_buffers()}
  x = feat.clone().requires_grad_()
  logits = net(x, o, depth, query.clone().to(DEV))
  loss = _loss(logits, labels.to(DEV))
  loss.backward()

  params = {k: v.detach().double().cpu().requires_grad_() for k, v in net.named_parameters()}
  xr = feat.detach().double().cpu().requires_grad_()
  q = query.numpy().copy()
  q[:, :3] = (q[:, :3] + 1.0) * np.float32(2 ** (depth - 1))        # OctreeInterp's rescaling
  want = OracleUNet(params, ref, nempty, running)(xr, depth, q)
  want_loss = _loss(want, labels)
  want_loss.backward()

  def rel(got, exp):
    return float((got.detach().double().cpu() - exp).abs().max() / exp.abs().max().clamp_min(1e-30))
  e = rel(logits, want.detach())
  say('   logits rel err %.2e   loss %.6f vs %.6f' % (e, float(loss), float(want_loss)))
  assert e < 1e-4
  assert abs(float(loss) - float(want_loss)) < 1e-5
  # Gradients.  A ReLU whose argument is within rounding of zero comes out on the other side
  # in fp32 than in fp64, and on the coarse levels (16 .. 60 rows) one such unit changes single
  # entries of a weight gradient by several per cent: with the fp32 convolutions' 4e-6 added
  # to the oracle's own layer outputs as noise, the oracle differs from itself by 7e-2 in the
  # largest entry of one layer's gradient.  So entries are not compared one by one: every
  # parameter's gradient is held in the L2 norm, all of them together more tightly, and half
  # of them (the median) to what rounding alone gives.
  def l2(got, exp):
    return float((got.detach().double().cpu() - exp).norm() / exp.norm().clamp_min(1e-30))
  errs, sq_err, sq_all = [], 0.0, 0.0
  for name, p in net.named_parameters():
    assert p.grad is not None, name
    exp = params[name].grad
    errs.append((l2(p.grad, exp), rel(p.grad, exp), name))
    sq_err += float((p.grad.detach().double().cpu() - exp).norm() ** 2)
    sq_all += float(exp.norm() ** 2)
  errs.sort(reverse=True)
  total = (sq_err / sq_all) ** 0.5
  median = sorted(e[1] for e in errs)[len(errs) // 2]
  e = l2(x.grad, xr.grad)
  say('   gradients, relative L2 error: all parameters %.2e, input %.2e, median of the per-parameter max-norm '
      'errors %.2e; largest: %s' % (total, e, median, ', '.join('%.1e (max %.1e) %s' % v for v in errs[:4])))
  # (measured: stored statistics 1.4e-5 .. 4.7e-5 in all, 1.6e-2 in the worst parameter; batch
  # statistics 1.7e-2 .. 2.3e-2 in all: every batch norm divides by the spread of 16 .. 128 rows)
  assert total < (1e-1 if training else 1e-3)
  assert errs[0][0] < (2e-1 if training else 5e-2), errs[0]
  assert median < (1e-1 if training else 1e-2)
  assert e < (1e-1 if training else 1e-2)


def _first_block_definition(net, feat, table, dtype):
  """conv1 of the net (3x3x3 convolution on the table, batch norm with the statistics of the batch,
  ReLU) in fp64 with plain torch indexing on the device, from the parameters and the input as the
  run in `dtype` sees them (rounded to it)."""
  W = net.conv1.conv.weights.detach().to(dtype).double()                  # (27, cin, cout)
  x = feat.to(dtype).double()
  rows = table.shape[0]
  z = torch.zeros(rows, W.shape[2], dtype=torch.float64, device=DEV)
  for r0 in range(0, rows, 1 << 18):
    ts = table[r0:r0 + (1 << 18)].long()
    for k in range(27):
      z[r0:r0 + ts.shape[0]] += (x[ts[:, k].clamp_min(0)] * (ts[:, k] >= 0).unsqueeze(1)) @ W[k]
  bn = net.conv1.bn
  mean, var = z.mean(0), z.var(0, unbiased=False)
  y = (z - mean) / torch.sqrt(var + bn.eps) * bn.weight.detach().to(dtype).double() + bn.bias.detach().to(dtype).double()
  return y.clamp_min(0)


def test_unet_full_size_bf16():
  """configs[4] at full size on its own kind of scene (floor, walls, 10 - 20 boxes per cloud): the
  output of the first block (all rows) against its fp64 definition in fp32 (1e-4) and bf16 (2e-2),
  then the whole net in bf16 against its fp32 run, and twice on the same inputs (same bits)."""
  depth, batch, n = 9, 8, 150000
  say('U-Net, 8 x 150 000 points of indoor-like scenes, depth 9, non-empty nodes')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.indoor_cloud, batch, 1004, n=n)
  o = Octree(depth, 2, batch_size=batch)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=batch))
  o.construct_all_neigh()
  feat = o.get_input_feature('ND', True)
  query = torch.cat([pts, bid.float().view(-1, 1)], 1).to(DEV)
  labels = torch.randint(0, 10, (query.shape[0],), generator=torch.Generator().manual_seed(5)).to(DEV)
  torch.manual_seed(0)
  net = UNet(feat.shape[1], 10, 'linear', True).to(DEV)
  say('   rows per depth', o.nnum_nempty.tolist())
  table = o._table(depth, '333', 1, True)
  res = {}
  for dtype in (torch.float32, torch.bfloat16):
    say('  ', dtype)
    net.zero_grad(set_to_none=True)
    m = net.to(dtype)
    with torch.no_grad():
      got = m.conv1(feat.to(dtype), o, depth).double()
      want = _first_block_definition(net, feat, table, dtype)
      scale = float(want.abs().max())
      err = float((got - want).abs().max()) / scale
      row = (got - want).abs().amax(1) / want.abs().amax(1).clamp_min(0.05 * scale)
      say('   first block, %d rows: rel err %.2e, worst row %.2e' % (got.shape[0], err, float(row.max())))
      tol = 1e-4 if dtype == torch.float32 else 2e-2
      assert err < tol and float(row.max()) < 4 * tol
      del got, want, row
    logits = m(feat.to(dtype), o, depth, query.clone())
    loss = _loss(logits.float(), labels)
    loss.backward()
    grads = {k: p.grad.detach().float().clone() for k, p in m.named_parameters()}
    assert logits.shape == (query.shape[0], 10) and logits.dtype == dtype
    assert torch.isfinite(logits.float()).all() and bool(torch.isfinite(loss))
    for k, gk in grads.items():
      assert torch.isfinite(gk).all(), k
    res[dtype] = (float(loss), grads)
    if dtype == torch.bfloat16:
      # No kernel of the path sums in an order that depends on timing: the same step again gives
      # the same bits, logits and every parameter gradient (a load waited for too early, the
      # kind of defect a handful of wrong rows comes from, shows here as a difference).
      m.zero_grad(set_to_none=True)
      again = m(feat.to(dtype), o, depth, query.clone())
      _loss(again.float(), labels).backward()
      assert torch.equal(again, logits), 'logits differ between two runs'
      diff = [k for k, p in m.named_parameters() if not torch.equal(p.grad.float(), grads[k])]
      assert not diff, ('gradients differ between two runs', diff[:6])
      del again
    net = m.float()
  l32, g32 = res[torch.float32]
  l16, g16 = res[torch.bfloat16]
  say('   loss fp32 %.5f  bf16 %.5f' % (l32, l16))
  assert abs(l32 - l16) < 2e-2 * abs(l32)
  a = torch.cat([g32[k].flatten() for k in sorted(g32)])
  b = torch.cat([g16[k].flatten() for k in sorted(g32)])
  cos = float((a.double() @ b.double()) / (a.double().norm() * b.double().norm()))
  say('   cosine of the full gradient vectors %.4f, norm ratio %.4f' % (cos, float(b.norm() / a.norm())))
  assert cos > 0.9


def test_residual_blocks_replay_from_a_hip_graph():
  """Forward + backward of a chain of residual blocks (3x3x3 convolutions, batch norm with running
  statistics and batch counter, ReLU, 1x1 projection of the shortcut) captured in a HIP graph after
  two eager steps: every replay gives the bits of an eager step, and the batch counters count the
  replays (they are incremented by a kernel, not by the host)."""
  from ocnn_amd.modules import OctreeResBlocks
  say('residual blocks from a hip graph')
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 2, 77, n=30000)
  o = Octree(7, 2, batch_size=2)
  o.build_octree(Points(pts.to(DEV), nrm.to(DEV), batch_id=bid.to(DEV), batch_size=2))
  o.construct_all_neigh()
  depth, dtype = 7, torch.bfloat16
  torch.manual_seed(3)
  net = OctreeResBlocks(32, 64, 2, bottleneck=1, nempty=True).to(DEV).to(dtype)
  rows = int(o.nnum_nempty[depth])
  x = torch.randn(rows, 32, device=DEV).to(dtype).requires_grad_()
  gout = torch.randn(rows, 64, device=DEV).to(dtype)
  params = [x] + list(net.parameters())
  counters = [m.num_batches_tracked for m in net.modules() if hasattr(m, 'num_batches_tracked')]
  assert len(counters) == 5

  def step():
    for p in params:
      p.grad = None
    out = net(x, o, depth)
    out.backward(gout)
    return out

  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    for _ in range(2):
      out = step()
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  want = [out.detach().clone()] + [p.grad.clone() for p in params]
  del out
  assert all(int(c) == 2 for c in counters)
  graph = torch.cuda.CUDAGraph()
  for p in params:
    p.grad = None
  with torch.cuda.graph(graph):
    out_g = net(x, o, depth)
    out_g.backward(gout)
  for replay in range(3):
    out_g.detach().zero_()
    for p in params:
      p.grad.zero_()
    (torch.randn(500, 64, device=DEV) @ torch.randn(64, 64, device=DEV)).sum().item()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    for a, b in zip(want, [out_g] + [p.grad for p in params]):
      assert torch.equal(a, b), replay
  assert all(int(c) == 2 + 3 for c in counters), [int(c) for c in counters]
