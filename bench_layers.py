"""Per-layer timings of the other layer configurations of the hot path on one
MI355X (the headline number is bench.py's; these lines are supporting data).

  config 2: depth-8 batch of 8 (100k points each), bf16: OctreeConv 2x2x2 stride 2
            64->128 (depth 8->7), OctreeDeconv 2x2x2 stride 2 128->64 (7->8),
            OctreeDWConv 3x3x3 on 128 channels at depth 7; also the 3x3x3 64->64 layer
            with nempty=True, and the pieces a U-Net adds around the convolutions (point
            interpolation at the 800k input points, 2x2x2 max pooling).
  config 3: batch of 4, depth 9, 250k points each (planes + spheres), bf16:
            OctreeConv 3x3x3 32->32 at depth 9 and 256->256 at depth 6; build_octree and
            construct_all_neigh on the 1M points.

  config 4: the U-Net's octree (batch of 8, 150k points each, depth 9), bf16: 3x3x3 and
            2x2x2 stride-2 layers of 96 / 128 channels on the non-empty nodes of depths 9 and
            8 (the tables the pair-plan kernels are for).
  config f4: the rest of the kernel-shape x stride grid on the depth-8 batch of config 2, bf16,
            64 channels: 3x3x3 stride 2 (conv and deconv), the axis kernels 3x1x1 and 3x3x1 at
            stride 1 and 2, 2x2x2 at stride 1, on all nodes and on non-empty nodes.
  config bn (not in the default set): batch norm + ReLU, forward + backward, on the tensors of
            the U-Net of config 4.

Every layer runs forward + backward through the module (autograd included); one JSON
line per layer: ms per fwd+bwd, effective TFLOP/s over non-empty neighbours, and the
rate at the algorithmic byte count as a fraction of 8 TB/s.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, 'ocnn-pytorch_amd')):
  if p not in sys.path:
    sys.path.insert(0, p)


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--steps', type=int, default=30)
  ap.add_argument('--warmup', type=int, default=5)
  ap.add_argument('--configs', default='2,3,4,f4')
  ap.add_argument('--scene', default='indoor', choices=['indoor', 'mixed'],
                  help="clouds of config 4: indoor-like scenes (the configuration's), or 3 spheres + 2 boxes")
  args = ap.parse_args()
  import torch
  from ocnn_amd import synthetic
  from ocnn_amd.nn import OctreeConv, OctreeDeconv, OctreeDWConv
  from ocnn_amd.octree import Octree, Points
  assert torch.cuda.is_available(), 'bench_layers.py needs a GPU'
  dev = 'cuda:0'
  torch.cuda.set_device(0)

  def build(cloud, batch, seed, n, depth):
    pts, nrm, bid = synthetic.batch_clouds(cloud, batch, seed, n=n)
    pc = Points(pts.to(dev), nrm.to(dev), batch_id=bid.to(dev), batch_size=batch)
    times = []
    for _ in range(3):
      o = Octree(depth, 2, batch_size=batch)
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      o.build_octree(pc)
      torch.cuda.synchronize()
      t1 = time.perf_counter()
      o.construct_all_neigh()
      torch.cuda.synchronize()
      times.append((t1 - t0, time.perf_counter() - t1))
    return o, min(t[0] for t in times) * 1e3, min(t[1] for t in times) * 1e3, int(pts.shape[0])

  def run(tag, mod, octree, depth, rows_in, cin, cout, table, dtype, dw=False):
    g = torch.Generator().manual_seed(7)
    mod = mod.to(dev).to(dtype)
    x = torch.randn(rows_in, cin, generator=g).to(dtype).to(dev).requires_grad_()
    out = mod(x, octree, depth)
    gout = torch.randn(out.shape, generator=g).to(dtype).to(dev)

    def step():
      x.grad = None
      mod.weights.grad = None
      mod(x, octree, depth).backward(gout)

    for _ in range(args.warmup):
      step()
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(args.steps):
      step()
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / args.steps
    rows, K = table.shape
    nnz = int((table >= 0).sum())
    flops = 6.0 * nnz * (cin if dw else cin * cout)
    es = 2
    if dw:
      bytes_ = 3 * (es * (rows_in * cin + rows * cin + K * cin) + 4 * rows * K)
    else:
      bytes_ = 3 * (es * (rows_in * cin + rows * cout) + 4 * rows * K) + 2 * es * K * cin * cout + 4 * K * cin * cout
    print(json.dumps({
        'layer': tag, 'dtype': str(dtype).replace('torch.', ''), 'rows_in': rows_in, 'rows_table': rows,
        'K': K, 'nnz': nnz, 'ms_fwd_bwd': ms, 'eff_tflops': flops / ms / 1e9,
        'frac_mfma_peak': flops / ms / 1e9 / 2500.0,
        'algorithmic_bytes': bytes_, 'frac_hbm_peak_at_algorithmic_bytes': bytes_ / ms / 1e6 / 8000.0,
    }), flush=True)

  def run_op(tag, step, bytes_, extra):
    for _ in range(args.warmup):
      step()
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(args.steps):
      step()
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / args.steps
    d = {'op': tag, 'ms_fwd_bwd': ms, 'algorithmic_bytes': bytes_,
         'frac_hbm_peak_at_algorithmic_bytes': bytes_ / ms / 1e6 / 8000.0}
    d.update(extra)
    print(json.dumps(d), flush=True)

  def ops(o, depth, pts, bid):
    """The pieces a U-Net adds around the convolutions: point interpolation of the output
    features, max pooling (non-empty nodes, as the networks use them)."""
    from ocnn_amd.nn import octree_linear_pts, octree_nearest_pts, octree_max_pool
    g = torch.Generator().manual_seed(9)
    rows = int(o.nnum_nempty[depth])
    q = torch.cat([(pts.to(dev) + 1.0) * (2 ** (depth - 1)), bid.to(dev).float().view(-1, 1)], 1)
    n = q.shape[0]
    for c, dt in ((64, torch.float32), (64, torch.bfloat16)):
      es = 4 if dt == torch.float32 else 2
      data = torch.randn(rows, c, generator=g).to(dt).to(dev).requires_grad_()
      gout = torch.randn(n, c, generator=g).to(dt).to(dev)
      for name, fn in (('linear', octree_linear_pts), ('nearest', octree_nearest_pts)):
        def step():
          data.grad = None
          fn(data, o, depth, q, nempty=True).backward(gout)
        run_op('interp %s %d ch d%d nempty %s' % (name, c, depth, str(dt).replace('torch.', '')), step,
               2 * (es * (n * c + rows * c) + 16 * n), {'points': n, 'rows': rows})
    data = torch.randn(rows, 64, generator=g).to(torch.bfloat16).to(dev).requires_grad_()
    prow = int(o.nnum_nempty[depth - 1])
    gout = torch.randn(prow, 64, generator=g).to(torch.bfloat16).to(dev)

    def step():
      data.grad = None
      octree_max_pool(data, o, depth, nempty=True).backward(gout)
    run_op('max pool 64 ch d%d->%d nempty bfloat16' % (depth, depth - 1), step,
           2 * 2 * (rows * 64 + prow * 64) + 2 * 8 * prow * 64, {'rows': rows, 'parents': prow})

  bf = torch.bfloat16
  if 'bn' in args.configs.split(','):
    # batch norm + ReLU, training mode, on the tensors of the U-Net of config 4 (rows of the non-empty
    # nodes of depths 9 .. 5 x the channels the net has there): forward 2 reads + 1 write, backward
    # 4 reads + 1 write of the tensor
    from ocnn_amd.nn import BatchNormRelu1d
    for rows, c in ((925113, 32), (925113, 96), (621985, 64), (621985, 96), (280645, 128), (83376, 256),
                    (21148, 256)):
      bn = BatchNormRelu1d(c, relu=True).to(dev).to(bf)
      x = torch.randn(rows, c, device=dev).to(bf).requires_grad_()
      g = torch.randn(rows, c, device=dev).to(bf)

      def step():
        x.grad = None
        bn(x).backward(g)
      run_op('batch norm + relu %d x %d bfloat16' % (rows, c), step, 8 * rows * c * 2, {'rows': rows, 'channels': c})
  if '2' in args.configs.split(','):
    o, b_ms, n_ms, npts = build(synthetic.mixed_cloud, 8, 1001, 100000, 8)
    print(json.dumps({'octree': 'config 2 (batch 8, depth 8)', 'points': npts, 'build_octree_ms': b_ms,
                      'construct_all_neigh_ms': n_ms, 'nnum': o.nnum.tolist(),
                      'nnum_nempty': o.nnum_nempty.tolist()}), flush=True)
    nn8, ne8, nn7, ne7 = int(o.nnum[8]), int(o.nnum_nempty[8]), int(o.nnum[7]), int(o.nnum_nempty[7])
    run('conv 2x2x2 s2 64->128 d8->7', OctreeConv(64, 128, [2], 2), o, 8, nn8, 64, 128,
        o._table(8, '222', 2, False), bf)
    run('deconv 2x2x2 s2 128->64 d7->8', OctreeDeconv(128, 64, [2], 2), o, 7, nn7, 128, 64,
        o._table(8, '222', 2, False), bf)
    run('dwconv 3x3x3 128 d7', OctreeDWConv(128, [3], 1), o, 7, nn7, 128, 128,
        o._table(7, '333', 1, False), bf, dw=True)
    run('conv 3x3x3 s1 64->64 d8 nempty', OctreeConv(64, 64, [3], 1, nempty=True), o, 8, ne8, 64, 64,
        o._table(8, '333', 1, True), bf)
    run('conv 3x3x3 s1 64->64 d8', OctreeConv(64, 64, [3], 1), o, 8, nn8, 64, 64,
        o._table(8, '333', 1, False), bf)
    pts, _, bid = synthetic.batch_clouds(synthetic.mixed_cloud, 8, 1001, n=100000)
    ops(o, 8, pts, bid)
    del o
  if '3' in args.configs.split(','):
    o, b_ms, n_ms, npts = build(synthetic.planes_cloud, 4, 1003, 250000, 9)
    print(json.dumps({'octree': 'config 3 (batch 4, depth 9)', 'points': npts, 'build_octree_ms': b_ms,
                      'construct_all_neigh_ms': n_ms, 'nnum': o.nnum.tolist(),
                      'nnum_nempty': o.nnum_nempty.tolist()}), flush=True)
    run('conv 3x3x3 s1 32->32 d9', OctreeConv(32, 32, [3], 1), o, 9, int(o.nnum[9]), 32, 32,
        o._table(9, '333', 1, False), bf)
    run('conv 3x3x3 s1 256->256 d6', OctreeConv(256, 256, [3], 1), o, 6, int(o.nnum[6]), 256, 256,
        o._table(6, '333', 1, False), bf)
  if 'f4' in args.configs.split(','):
    o, b_ms, n_ms, npts = build(synthetic.mixed_cloud, 8, 1001, 100000, 8)
    print(json.dumps({'octree': 'config f4 (batch 8, depth 8)', 'points': npts, 'build_octree_ms': b_ms,
                      'construct_all_neigh_ms': n_ms}), flush=True)
    C = 64
    for ks, stride in (([3, 3, 3], 2), ([3, 1, 1], 1), ([3, 1, 1], 2), ([3, 3, 1], 1), ([3, 3, 1], 2), ([2, 2, 2], 1)):
      kern = ''.join(str(k) for k in ks)
      for ne in (False, True):
        for kind, Mod in (('conv', OctreeConv), ('deconv', OctreeDeconv)):
          if kind == 'deconv' and stride == 1:
            continue
          d = 8 if kind == 'conv' else 7
          rows_in = int(o.nnum_nempty[d] if ne else o.nnum[d])
          run('%s %s s%d %d->%d d%d%s' % (kind, 'x'.join(kern), stride, C, C, d, ' nempty' if ne else ''),
              Mod(C, C, ks, stride, nempty=ne), o, d, rows_in, C, C,
              o._table(d if kind == 'conv' else d + 1, kern, stride, ne), bf)
    del o
  if '4' in args.configs.split(','):
    # the U-Net's octree (config 4: batch 8, 150k points each, depth 9), layers on the non-empty
    # nodes of depths 9 and 8, where 14 % / 25 % of the table entries hold a neighbour
    o, b_ms, n_ms, npts = build(synthetic.indoor_cloud if args.scene == 'indoor' else synthetic.mixed_cloud, 8, 1004,
                                150000, 9)
    print(json.dumps({'octree': 'config 4 (batch 8, depth 9, %s scenes)' % args.scene, 'points': npts, 'build_octree_ms': b_ms,
                      'construct_all_neigh_ms': n_ms, 'nnum_nempty': o.nnum_nempty.tolist()}), flush=True)
    ne9, ne8 = int(o.nnum_nempty[9]), int(o.nnum_nempty[8])
    run('conv 3x3x3 s1 96->96 d9 nempty', OctreeConv(96, 96, [3], 1, nempty=True), o, 9, ne9, 96, 96,
        o._table(9, '333', 1, True), bf)
    run('conv 3x3x3 s1 96->96 d8 nempty', OctreeConv(96, 96, [3], 1, nempty=True), o, 8, ne8, 96, 96,
        o._table(8, '333', 1, True), bf)
    run('conv 3x3x3 s1 128->96 d9 nempty', OctreeConv(128, 96, [3], 1, nempty=True), o, 9, ne9, 128, 96,
        o._table(9, '333', 1, True), bf)
    # the coarse levels of the same net (encoder 64 / 128 / 256 channels at depths 7 / 6 / 5, decoder 256 / 128
    # at depths 6 / 7): few rows, many channels
    for d, c in ((7, 64), (7, 128), (6, 128), (6, 256), (5, 256)):
      run('conv 3x3x3 s1 %d->%d d%d nempty' % (c, c, d), OctreeConv(c, c, [3], 1, nempty=True), o, d,
          int(o.nnum_nempty[d]), c, c, o._table(d, '333', 1, True), bf)
    run('conv 2x2x2 s2 96->96 d9->8 nempty', OctreeConv(96, 96, [2], 2, nempty=True), o, 9, ne9, 96, 96,
        o._table(9, '222', 2, True), bf)
    run('deconv 2x2x2 s2 96->96 d8->9 nempty', OctreeDeconv(96, 96, [2], 2, nempty=True), o, 8, ne8, 96, 96,
        o._table(9, '222', 2, True), bf)


if __name__ == '__main__':
  main()
