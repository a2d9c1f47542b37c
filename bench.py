"""Benchmark of the octree sparse-convolution hot path on one MI355X.

One step = OctreeConv 3x3x3 stride 1, 64 -> 64 channels, forward + backward
(data and weight gradients) at depth 8 over a batch of 8 synthetic octrees
(100k surface points each), fp16 features/weights with fp32 accumulation.
Inputs (octree, tables, features) are resident in HBM before the timed region.

Prints one JSON line; `value` is effective TFLOP/s counting only non-empty
neighbours (6 * nnz * Cin * Cout per step).
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

PEAK_MFMA_16BIT_TFLOPS = 2500.0     # MI355X dense bf16 / fp16
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the gather-GEMM kernel at the default workload (fp16, depth 8,
# batch 8), from rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a 1 GiB copy; None for
# any other workload.  The summary under profiles/ gives the counter readings.
TRAFFIC_GATHER_DEFAULT = int((209100 * 2.0 + 235970 * 1.0) * 1024)


def parse():
  ap = argparse.ArgumentParser()
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=50)
  ap.add_argument('--warmup', type=int, default=10)
  ap.add_argument('--dtype', default='fp16', choices=['fp16', 'bf16'])
  ap.add_argument('--nempty', type=int, default=0)
  ap.add_argument('--depth', type=int, default=8)
  ap.add_argument('--batch', type=int, default=8)
  ap.add_argument('--points', type=int, default=100000)
  ap.add_argument('--channels', type=int, default=64)
  ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
  ap.add_argument('--cpu-rows', type=int, default=262144)
  ap.add_argument('--only', default='all', choices=['all', 'fwd', 'bwd_data', 'wgrad'],
                  help='run a single pass per step (for counter collection); the JSON line is '
                       'then not a benchmark result')
  ap.add_argument('--calib', action='store_true',
                  help='also run one 1 GiB device copy, to scale FETCH_SIZE / WRITE_SIZE')
  return ap.parse_args()


class KernelTimer:
  """Brackets every call of one library entry point with events on the stream
  the kernels are launched on (torch's current stream)."""

  def __init__(self, torch, module, name):
    self.torch, self.module, self.name = torch, module, name
    self.orig = getattr(module, name)
    self.events = []
    self.enabled = False

    def wrapped(*a, **kw):
      if not self.enabled:
        return self.orig(*a, **kw)
      s = torch.cuda.Event(enable_timing=True)
      e = torch.cuda.Event(enable_timing=True)
      s.record()
      out = self.orig(*a, **kw)
      e.record()
      self.events.append((s, e))
      return out

    setattr(module, name, wrapped)

  def mean_ms(self):
    if not self.events:
      return None
    return sum(s.elapsed_time(e) for s, e in self.events) / len(self.events)

  def count(self):
    return len(self.events)


def cpu_baseline(torch, table32, rows_in, cin, cout, sample_rows):
  """Times the reference's CPU execution form (chunked gather -> mm ->
  scatter_add, oracle.conv_ref.BlockGemmCPU, fp32) on the first `sample_rows`
  rows of the same neighbour table, forward + both gradients."""
  from oracle.conv_ref import BlockGemmCPU
  g = torch.Generator().manual_seed(7)
  table = table32[:sample_rows].long().cpu()
  data = torch.randn(rows_in, cin, generator=g)
  W = torch.randn(27, cin, cout, generator=g) / 40.0
  grad = torch.randn(table.shape[0], cout, generator=g)

  def one(tab, gr):
    eng = BlockGemmCPU(tab, cin)
    eng.forward(data, W)
    eng.backward(gr, W, rows_in)
    eng.weight(data, gr, tuple(W.shape))

  one(table[:8192], grad[:8192])                      # warm-up
  t0 = time.perf_counter()
  one(table, grad)
  dt = time.perf_counter() - t0
  nnz = int((table >= 0).sum())
  return {
      'value': 6.0 * nnz * cin * cout / dt / 1e12,
      'unit': 'TFLOP/s',
      'cores': torch.get_num_threads(),
      'kind': 'port',
      'sample': 'first {} of {} table rows, fp32, fwd+bwd-data+bwd-weight, {:.2f} s; '
                'host cpu_count={} affinity={}'.format(
                    table.shape[0], table32.shape[0], dt, os.cpu_count(),
                    len(os.sched_getaffinity(0))),
      'ms_per_step_extrapolated': dt * 1e3 * table32.shape[0] / table.shape[0],
  }


def main():
  args = parse()
  if args.gpus != 1:
    print('bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1',
          file=sys.stderr)
    sys.exit(2)
  import torch
  import ocnn_amd
  from ocnn_amd import synthetic
  from ocnn_amd.nn import OctreeConv
  import importlib
  conv_mod = importlib.import_module('ocnn_amd.nn.octree_conv')
  from ocnn_amd.octree import Octree, Points

  assert torch.cuda.is_available(), 'bench.py needs a GPU'
  dev = 'cuda:0'
  torch.cuda.set_device(0)
  dtype = torch.float16 if args.dtype == 'fp16' else torch.bfloat16
  C = args.channels
  nempty = bool(args.nempty)

  # ---- inputs: synthetic clouds -> octree (timed separately) ----------------
  pts, nrm, bid = synthetic.batch_clouds(synthetic.mixed_cloud, args.batch, 1001, n=args.points)
  pc = Points(pts.to(dev), nrm.to(dev), batch_id=bid.to(dev) if args.batch > 1 else None,
              batch_size=args.batch)

  def build():
    o = Octree(args.depth, 2, batch_size=args.batch)
    o.build_octree(pc)
    torch.cuda.synchronize()
    t = time.perf_counter()
    o.construct_all_neigh()
    torch.cuda.synchronize()
    return o, time.perf_counter() - t

  build()                                              # warm-up (first-use costs)
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  octree, neigh_s = build()
  build_s = time.perf_counter() - t0 - neigh_s

  depth = args.depth
  table = octree._table(depth, '333', 1, nempty)
  rows = table.shape[0]
  nnz = int((table >= 0).sum())
  g = torch.Generator().manual_seed(1001)
  conv = OctreeConv(C, C, [3], 1, nempty=nempty)
  with torch.no_grad():
    bound = 1.0 / (27 * C) ** 0.5                      # Kaiming-uniform bound
    conv.weights.copy_((torch.rand(conv.weights.shape, generator=g) * 2 - 1) * bound)
  conv = conv.to(dev).to(dtype)
  x = torch.randn(rows, C, generator=g).to(dtype).to(dev).requires_grad_()
  gout = torch.randn(rows, C, generator=g).to(dtype).to(dev)

  t_gather = KernelTimer(torch, conv_mod, 'conv_gather')
  t_wgrad = KernelTimer(torch, conv_mod, 'conv_wgrad')

  eng = conv_mod._OctreeConv(C, C, [3], 1, nempty)
  eng.setup(octree, depth)
  w_cast = conv.weights.detach()

  def step():
    if args.only == 'fwd':
      eng.forward_gemm(x.detach(), w_cast)
    elif args.only == 'bwd_data':
      eng.backward_gemm(gout, w_cast)
    elif args.only == 'wgrad':
      eng.weight_gemm(x.detach(), gout)
    else:
      x.grad = None
      conv.weights.grad = None
      out = conv(x, octree, depth)
      out.backward(gout)

  if args.calib:
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  t_gather.enabled = t_wgrad.enabled = True
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step()
  torch.cuda.synchronize()
  dt = time.perf_counter() - t0
  ms = dt * 1e3 / args.steps

  flops_step = 6.0 * nnz * C * C
  gather_ms = t_gather.mean_ms() or float('nan')
  wgrad_ms = t_wgrad.mean_ms() or float('nan')
  flops_launch = 2.0 * nnz * C * C
  achieved = flops_launch / (gather_ms * 1e-3) / 1e12
  es = 2                                               # bytes per feature element
  bytes_gather = es * (rows * C + rows * C + 27 * C * C) + 4 * rows * 27
  bytes_wgrad = es * (rows * C + rows * C) + 4 * rows * 27 + 4 * 27 * C * C

  default_workload = (args.depth, args.batch, args.points, C, nempty) == (8, 8, 100000, 64, False)
  TRAFFIC_GATHER_BYTES = TRAFFIC_GATHER_DEFAULT if default_workload else None
  result = {
      'metric': 'OctreeConv 3x3x3 64->64 fwd+bwd at depth 8 (batch 8): effective TFLOP/s '
                'over non-empty neighbours',
      'value': flops_step / dt * args.steps / 1e12,
      'unit': 'TFLOP/s',
      'n_gpus': 1,
      'steps': args.steps,
      'warmup': args.warmup,
      'ms_per_step': ms,
      'higher_is_better': True,
      'scaling': 'weak',
      'vs_baseline': None,
      'dtype': args.dtype + ' (fp32 accumulate)',
      'data': 'synthetic',
      'config': {
          'workload': 'configs[1]: batch {} octrees, depth {}, full_depth 2, {} surface points '
                      'each (3 spheres + 2 boxes); OctreeConv 3x3x3 stride 1 {}->{} {}, '
                      'nempty={}; forward + backward'.format(
                          args.batch, depth, args.points, C, C, args.dtype, nempty),
          'rows': rows, 'nnz': nnz, 'valid_per_row': nnz / rows,
      },
      'roofline': {
          'kernel': 'conv_gather_rw_kernel (forward and data gradient; mean of both launches, '
                    'each bracketed with its weight-pack pre-pass)',
          'bound': 'mfma',
          'achieved': achieved,
          'peak': PEAK_MFMA_16BIT_TFLOPS,
          'unit': 'TFLOP/s',
          'frac': achieved / PEAK_MFMA_16BIT_TFLOPS,
          'traffic': TRAFFIC_GATHER_BYTES,
          'launches': t_gather.count(),
          'avg_launch_ms': gather_ms,
          'algorithmic_flops_per_launch': flops_launch,
          'algorithmic_bytes_per_launch': bytes_gather,
          'hbm_frac_at_algorithmic_bytes': bytes_gather / (gather_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
      },
      'kernels': {
          'conv_gather_ms': gather_ms,
          'conv_wgrad_ms': wgrad_ms,
          'conv_wgrad_tflops': flops_launch / (wgrad_ms * 1e-3) / 1e12,
          'conv_wgrad_algorithmic_bytes': bytes_wgrad,
          'sustained_mfma_note': 'v_mfma_f32_32x32x16_f16 alone sustains 1.67 PFLOP/s on this part with '
                                 'random operands (2.38 with constant ones): clocks drop under load',
          'fraction_of_mfma_peak_whole_step': flops_step / (ms * 1e-3) / 1e12 / PEAK_MFMA_16BIT_TFLOPS,
      },
      'octree': {
          'points': int(pts.shape[0]),
          'build_octree_ms': build_s * 1e3,
          'construct_all_neigh_ms': neigh_s * 1e3,
          'nnum': octree.nnum.tolist(),
          'nnum_nempty': octree.nnum_nempty.tolist(),
      },
  }
  if args.only != 'all':
    result['note'] = 'single-pass run (--only {}): not a benchmark result'.format(args.only)
  if not args.no_cpu:
    result['cpu_baseline'] = cpu_baseline(torch, table, x.shape[0], C, C, args.cpu_rows)
  print(json.dumps(result))


if __name__ == '__main__':
  main()
