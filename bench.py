"""Benchmark of the octree sparse-convolution hot path on one MI355X.

One step = OctreeConv 3x3x3 stride 1, 64 -> 64 channels, forward + backward (data and weight
gradients) through the module at depth 8 over a batch of 8 synthetic octrees (100k surface
points each), bf16 features / weights with fp32 accumulation (configs[1] of BASELINE.json, in
the dtype its target sentence names; the same step in fp16 is reported beside it).  Inputs
(octree, tables, tile plans, features) are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is effective TFLOP/s counting only non-empty neighbours
(6 * nnz * Cin * Cout per step).  Beside it: the dominant kernel against its roofline, what
the part itself sustains (MFMA rate with N(0, 1) operands), what a step costs when every step
brings a new octree (build, tables, plans), compact records of the layers of configs[2] and
configs[3], and the reference's CPU execution form timed on the host cores.
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, 'ocnn-pytorch_amd')):
  if p not in sys.path:
    sys.path.insert(0, p)

from bench_common import PEAK_HBM_GBS, PEAK_MFMA_16BIT_TFLOPS, build_octree, time_layer   # noqa: E402

# HBM bytes per launch of the gather-GEMM kernel at the default workload, from the rocprofv3
# FETCH_SIZE / WRITE_SIZE passes summarised in this file under profiles/ (not measured by this
# run: counters need the profiler); None for any other workload.
TRAFFIC_SOURCE = 'profiles/conv_kernels_counters_depth8_c64_bf16.txt'
TRAFFIC_GATHER_DEFAULT = int((208782 * 2.0 + 235796 * 1.0) * 1024)


def parse():
  ap = argparse.ArgumentParser()
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=50)
  ap.add_argument('--warmup', type=int, default=10)
  ap.add_argument('--dtype', default='bf16', choices=['fp16', 'bf16'])
  ap.add_argument('--nempty', type=int, default=0)
  ap.add_argument('--depth', type=int, default=8)
  ap.add_argument('--batch', type=int, default=8)
  ap.add_argument('--points', type=int, default=100000)
  ap.add_argument('--channels', type=int, default=64)
  ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
  ap.add_argument('--no-extras', action='store_true',
                  help='headline step only: no second dtype, other layers, probes or fresh-octree steps')
  ap.add_argument('--cpu-rows', type=int, default=524288)
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

  def reset(self):
    self.events = []


def cpu_baseline(torch, table32, rows_in, cin, cout, sample_rows):
  """Times the reference's CPU execution form (chunked gather -> mm -> scatter_add,
  oracle.conv_ref.BlockGemmCPU, fp32) on the first `sample_rows` rows of the same neighbour
  table, forward + both gradients: one warm-up, three timed runs, the median."""
  from oracle.conv_ref import BlockGemmCPU
  g = torch.Generator().manual_seed(7)
  table = table32[:sample_rows].long().cpu()
  data = torch.randn(rows_in, cin, generator=g)
  W = torch.randn(27, cin, cout, generator=g) / 40.0
  grad = torch.randn(table.shape[0], cout, generator=g)

  def one():
    t0 = time.perf_counter()
    eng = BlockGemmCPU(table, cin)
    eng.forward(data, W)
    eng.backward(grad, W, rows_in)
    eng.weight(data, grad, tuple(W.shape))
    return time.perf_counter() - t0

  one()                                               # warm-up
  runs = [one() for _ in range(3)]
  dt = statistics.median(runs)
  nnz = int((table >= 0).sum())
  return {
      'value': 6.0 * nnz * cin * cout / dt / 1e12,
      'unit': 'TFLOP/s',
      'cores': torch.get_num_threads(),
      'kind': 'port',
      'sample': 'first {} of {} table rows, fp32, fwd+bwd-data+bwd-weight; 1 warm-up + 3 timed runs '
                '({}) s, median {:.2f} s; host cpu_count={} affinity={}'.format(
                    table.shape[0], table32.shape[0], ', '.join('%.2f' % r for r in runs), dt, os.cpu_count(),
                    len(os.sched_getaffinity(0))),
      'ms_per_step_extrapolated': dt * 1e3 * table32.shape[0] / table.shape[0],
  }


def cpu_baseline_octree(pts, nrm, bid, depth, batch):
  """The octree construction and the neighbour search of the same clouds on the host: the oracle's
  numpy restatement of ocnn/octree/octree.py:201-287 and :404-446 (one thread), one run each."""
  from oracle import octree_ref
  t0 = time.perf_counter()
  o, _ = octree_ref.build_octree(pts.numpy(), nrm.numpy(), None, None if bid is None else bid.numpy(), depth, 2,
                                 batch)
  t1 = time.perf_counter()
  octree_ref.construct_all_neigh(o)
  t2 = time.perf_counter()
  return {'build_octree_ms': (t1 - t0) * 1e3, 'construct_all_neigh_ms': (t2 - t1) * 1e3, 'cores': 1, 'kind': 'port',
          'sample': 'all {} points, depth {}, batch {}; numpy, one run'.format(pts.shape[0], depth, batch)}


def main():
  args = parse()
  if args.gpus != 1:
    print('bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1',
          file=sys.stderr)
    sys.exit(2)
  import torch
  import ocnn_amd
  from ocnn_amd import synthetic
  from ocnn_amd.nn import OctreeConv, OctreeDeconv, OctreeDWConv
  import importlib
  conv_mod = importlib.import_module('ocnn_amd.nn.octree_conv')
  from ocnn_amd.octree import Octree, Points
  from ocnn_amd.octree.octree import TilePlan

  assert torch.cuda.is_available(), 'bench.py needs a GPU'
  dev = 'cuda:0'
  torch.cuda.set_device(0)
  DT = {'fp16': torch.float16, 'bf16': torch.bfloat16}
  dtype = DT[args.dtype]
  C = args.channels
  nempty = bool(args.nempty)
  depth = args.depth
  extras = not args.no_extras and args.only == 'all'

  # ---- inputs: synthetic clouds -> octree (timed separately) ----------------
  build_octree(torch, synthetic, Octree, Points, synthetic.mixed_cloud, args.batch, 1001, args.points, depth, dev, 1)
  octree, build_ms, neigh_ms, pts, bid, pc = build_octree(torch, synthetic, Octree, Points, synthetic.mixed_cloud,
                                                          args.batch, 1001, args.points, depth, dev)
  # every table written once, the parents' rows and the children read once
  neigh_bytes = sum(int(octree.nnum[d]) * 27 * 4 + int(octree.nnum_nempty[d - 1]) * 27 * 4 + int(octree.nnum[d - 1]) * 4
                    for d in range(1, depth + 1))
  table = octree._table(depth, '333', 1, nempty)
  rows = table.shape[0]
  nnz = int((table >= 0).sum())
  plan_ms = []
  for _ in range(3):                                   # one tile plan, built alone (once per octree and table)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    TilePlan(table)
    torch.cuda.synchronize()
    plan_ms.append((time.perf_counter() - t0) * 1e3)

  g = torch.Generator().manual_seed(1001)
  conv = OctreeConv(C, C, [3], 1, nempty=nempty)
  with torch.no_grad():
    bound = 1.0 / (27 * C) ** 0.5                      # Kaiming-uniform bound
    conv.weights.copy_((torch.rand(conv.weights.shape, generator=g) * 2 - 1) * bound)
  x_dev = torch.randn(rows, C, generator=g).to(dev)
  gout_dev = torch.randn(rows, C, generator=g).to(dev)

  t_gather = KernelTimer(torch, conv_mod, 'conv_gather')
  t_wgrad = KernelTimer(torch, conv_mod, 'conv_wgrad')
  eng = conv_mod._OctreeConv(C, C, [3], 1, nempty)
  eng.setup(octree, depth)

  def make_step(dt, oct=octree, only='all'):
    """The step closure of the layer in dtype `dt` on octree `oct`; all its tensors on the device."""
    m = OctreeConv(C, C, [3], 1, nempty=nempty)
    with torch.no_grad():
      m.weights.copy_(conv.weights)
    m = m.to(dev).to(dt)
    x = x_dev.to(dt).requires_grad_()
    gout = gout_dev.to(dt)
    w_cast = m.weights.detach()

    def step():
      if only == 'fwd':
        eng.forward_gemm(x.detach(), w_cast)
      elif only == 'bwd_data':
        eng.backward_gemm(gout, w_cast)
      elif only == 'wgrad':
        eng.weight_gemm(x.detach(), gout)
      else:
        x.grad = None
        m.weights.grad = None
        m(x, oct, depth).backward(gout)
    return step

  def run_steps(step, steps, warmup):
    """`warmup` untimed steps, then `steps` timed ones between synchronisations: ms per step,
    and the mean launch times of the two kernel families (events around every launch)."""
    for _ in range(warmup):
      step()
    torch.cuda.synchronize()
    t_gather.reset()
    t_wgrad.reset()
    t_gather.enabled = t_wgrad.enabled = True
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
      step()
      marks[i + 1].record()
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    t_gather.enabled = t_wgrad.enabled = False
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))
    run_steps.median_ms = per_step[len(per_step) // 2] if per_step else float('nan')
    return dt_s * 1e3 / steps, t_gather.mean_ms(), t_wgrad.mean_ms(), t_gather.count()

  def timed_steps(dt, steps, warmup, oct=octree, only='all'):
    return run_steps(make_step(dt, oct, only), steps, warmup)

  if args.calib:
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst

  # ---- from a cold start: the first steps, in blocks of five ----------------------
  # The step time falls over the first 30 ms or so of sustained work (1.21 -> 1.03 ms here;
  # it does again after a second of idling, and also right after 50 ms of matrix work that
  # touches no memory: it is the memory side of the chip that ramps).  The reference times
  # its layers with triton.testing.do_bench, 25 ms of warm-up before 100 ms of repetitions
  # (test/benchmark_conv.py:115,131).  This section shows the ramp and leaves the chip where
  # such a warm-up would; the W warm-up steps and the K timed steps of the contract follow.
  headline = make_step(dtype, only=args.only)
  cold = []
  if extras:
    headline()                                         # first call: module load, allocations, the plan
    torch.cuda.synchronize()
    time.sleep(1.0)                                    # from idle
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(9)]
    marks[0].record()
    for b in range(8):
      for _ in range(5):
        headline()
      marks[b + 1].record()
    torch.cuda.synchronize()
    cold = [marks[b].elapsed_time(marks[b + 1]) / 5 for b in range(8)]

  # ---- the headline step: W warm-up steps, K timed steps ---------------------------
  ms, gather_ms, wgrad_ms, n_gather = run_steps(headline, args.steps, args.warmup)
  median_ms = run_steps.median_ms
  gather_ms = gather_ms or float('nan')
  wgrad_ms = wgrad_ms or float('nan')
  flops_step = 6.0 * nnz * C * C
  flops_launch = 2.0 * nnz * C * C
  achieved = flops_launch / (gather_ms * 1e-3) / 1e12
  es = 2                                               # bytes per feature element
  bytes_gather = es * (rows * C + rows * C + 27 * C * C) + 4 * rows * 27
  bytes_wgrad = es * (rows * C + rows * C) + 4 * rows * 27 + 4 * 27 * C * C
  default_workload = (depth, args.batch, args.points, C, nempty) == (8, 8, 100000, 64, False)

  result = {
      'metric': 'OctreeConv 3x3x3 64->64 fwd+bwd at depth 8 (batch 8): effective TFLOP/s '
                'over non-empty neighbours',
      'value': flops_step / (ms * 1e-3) / 1e12,
      'unit': 'TFLOP/s',
      'n_gpus': 1,
      'steps': args.steps,
      'warmup': args.warmup,
      'ms_per_step': ms,
      'ms_per_step_median': median_ms,
      # every untimed step of the layer before the timed ones: the first call, the cold-start series and
      # the W warm-up steps (the timed steps follow them without a gap: a fully ramped figure)
      'untimed_steps_before_timing': (41 if extras else 0) + args.warmup,
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
      'fraction_of_mfma_peak_whole_step': flops_step / (ms * 1e-3) / 1e12 / PEAK_MFMA_16BIT_TFLOPS,
      'roofline': {
          'kernel': 'conv_gather_rw_kernel (forward and data gradient; mean of both launches, '
                    'each bracketed with its weight-pack pre-pass)',
          'bound': 'mfma',
          'achieved': achieved,
          'peak': PEAK_MFMA_16BIT_TFLOPS,
          'unit': 'TFLOP/s',
          'frac': achieved / PEAK_MFMA_16BIT_TFLOPS,
          'traffic': TRAFFIC_GATHER_DEFAULT if default_workload else None,
          'traffic_source': (TRAFFIC_SOURCE + ' (rocprofv3 FETCH_SIZE / WRITE_SIZE of an earlier run of this '
                             'command with --no-extras --calib, bf16; not measured by this run)')
          if default_workload else None,
          'launches': n_gather,
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
      },
      'octree': {
          'points': int(pts.shape[0]),
          'build_octree_ms': build_ms,
          'construct_all_neigh_ms': neigh_ms,
          'construct_all_neigh_algorithmic_bytes': neigh_bytes,
          'construct_all_neigh_hbm_frac': neigh_bytes / (neigh_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
          'tile_plan_ms_per_table': min(plan_ms),
          'nnum': octree.nnum.tolist(),
          'nnum_nempty': octree.nnum_nempty.tolist(),
      },
  }
  if args.only != 'all':
    result['note'] = 'single-pass run (--only {}): not a benchmark result'.format(args.only)

  if extras:
    result['cold_start'] = {'ms_per_step_blocks_of_5': [round(v, 4) for v in cold],
                            'note': '40 steps from an idle GPU (events every 5 steps), run right before the W warm-up '
                                    'steps: the step time falls for about 30 ms of sustained work before it settles'}
    # ---- the same step in the other 16-bit type ------------------------------
    other = 'fp16' if args.dtype == 'bf16' else 'bf16'
    oms, ogm, owm, _ = timed_steps(DT[other], args.steps, args.warmup)
    result['other_dtype'] = {'dtype': other, 'ms_per_step': oms, 'value': flops_step / (oms * 1e-3) / 1e12,
                             'conv_gather_ms': ogm, 'conv_wgrad_ms': owm,
                             'fraction_of_mfma_peak_whole_step': flops_step / (oms * 1e-3) / 1e12 /
                             PEAK_MFMA_16BIT_TFLOPS}

    # ---- what the part sustains: v_mfma_f32_32x32x16 alone, all CUs ----------
    try:
      import bench_probe as probe
      sustained = {k: probe.mfma_rate(dtype, k, 20000)['tflops'] for k in ('constant', 'normal')}
      alone, mixed = probe.mfma_mix(False), probe.mfma_mix(True)
      result['mfma_sustained'] = {
          'tflops_constant_operands': sustained['constant'], 'tflops_normal_operands': sustained['normal'],
          'two_chains_alone': {k: round(alone[k], 3) for k in ('tflops', 'ticks_per_mfma', 'ns_per_mfma', 'ghz')},
          'two_chains_with_gather_kernel_side_work': {k: round(mixed[k], 3) for k in
                                                      ('tflops', 'ticks_per_mfma', 'ns_per_mfma', 'ghz')},
          'gather_kernel_ns_per_mfma': gather_ms * 1e6 / (-(-rows // 128) / 256.0 * 224.0),
          'note': 'v_mfma_f32_32x32x16 back to back on every SIMD, {}: clocks fall under matrix load with '
                  'random operands, so this, not the published peak, bounds any kernel on N(0,1) data'.format(
                      args.dtype),
          'step_fraction_of_sustained_normal': flops_step / (ms * 1e-3) / 1e12 / sustained['normal'],
          'gather_kernel_dense_fraction_of_sustained_normal':
              (2.0 * rows * 28 * C * C / (gather_ms * 1e-3) / 1e12) / sustained['normal'],
      }
    except Exception as e:                              # the probe library is optional
      result['mfma_sustained'] = {'error': repr(e)}

    # ---- a new octree every step, as in training: build, tables, plans, step ---
    fresh = []
    for _ in range(3):
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      o = Octree(depth, 2, batch_size=args.batch)
      o.build_octree(pc)
      o.construct_all_neigh()
      torch.cuda.synchronize()
      t1 = time.perf_counter()
      fms, _, _, _ = timed_steps(dtype, 1, 0, oct=o)
      fresh.append(((t1 - t0) * 1e3, fms))
    fresh.sort(key=lambda v: v[0] + v[1])
    result['fresh_octree'] = {'build_and_tables_ms': fresh[1][0], 'first_step_with_plan_build_ms': fresh[1][1],
                              'note': 'median of 3; the step includes the tile plan of its table (built once per '
                                      'octree and table, shared by every layer and pass that uses the table)'}

    # ---- the layers of configs[2] and configs[3], bf16, forward + backward -----
    bf = torch.bfloat16
    ks, kw = min(args.steps, 20), min(args.warmup, 5)
    layers = []
    nn8, ne8, nn7 = int(octree.nnum[8]), int(octree.nnum_nempty[8]), int(octree.nnum[7])
    run = lambda *a, **k: layers.append(time_layer(torch, *a, steps=ks, warmup=kw, dev=dev, **k))
    if default_workload:
      run('configs[2] conv 2x2x2 s2 64->128 d8->7', OctreeConv(64, 128, [2], 2), octree, 8, nn8, 64, 128,
          octree._table(8, '222', 2, False), bf)
      run('configs[2] deconv 2x2x2 s2 128->64 d7->8', OctreeDeconv(128, 64, [2], 2), octree, 7, nn7, 128, 64,
          octree._table(8, '222', 2, False), bf)
      run('configs[2] dwconv 3x3x3 128 d7', OctreeDWConv(128, [3], 1), octree, 7, nn7, 128, 128,
          octree._table(7, '333', 1, False), bf, dw=True)
      run('configs[1] nempty=True: conv 3x3x3 s1 64->64 d8', OctreeConv(64, 64, [3], 1, nempty=True), octree, 8, ne8,
          64, 64, octree._table(8, '333', 1, True), bf)
      o3, b3, n3, p3, _, _ = build_octree(torch, synthetic, Octree, Points, synthetic.planes_cloud, 4, 1003, 250000,
                                          9, dev)
      run('configs[3] conv 3x3x3 s1 32->32 d9', OctreeConv(32, 32, [3], 1), o3, 9, int(o3.nnum[9]), 32, 32,
          o3._table(9, '333', 1, False), bf)
      run('configs[3] conv 3x3x3 s1 256->256 d6', OctreeConv(256, 256, [3], 1), o3, 6, int(o3.nnum[6]), 256, 256,
          o3._table(6, '333', 1, False), bf)
      result['configs3_octree'] = {'points': int(p3.shape[0]), 'build_octree_ms': b3, 'construct_all_neigh_ms': n3,
                                   'nnum_depth9': int(o3.nnum[9]), 'nnum_nempty_depth9': int(o3.nnum_nempty[9])}
      del o3
    result['other_layers'] = [
        {'layer': r['layer'], 'ms_fwd_bwd': round(r['ms_fwd_bwd'], 4), 'eff_tflops': round(r['eff_tflops'], 1),
         'pct_mfma_peak': round(100 * r['frac_mfma_peak'], 2),
         'pct_hbm_peak': round(100 * r['frac_hbm_peak_at_algorithmic_bytes'], 1)} for r in layers]

  if extras and default_workload:
    # ---- configs[4]: the reference's segmentation U-Net end to end (bench_unet.py) ----------
    try:
      import bench_unet
      u = bench_unet.run(['--steps', '10', '--warmup', '5', '--fresh', '1'])
      result['configs4_unet'] = {k: u[k] for k in ('net', 'scene', 'ms_per_step', 'ms_octree_build_and_tables',
                                                   'ms_first_step_on_a_fresh_octree',
                                                   'ms_per_step_new_octree_built_on_a_side_stream', 'dtype', 'nempty', 'batch',
                                                   'points', 'depth', 'rows_per_depth', 'parameters')}
      result['configs4_unet']['scene_note'] = ('indoor: floor, walls and 10 - 20 boxes per cloud, the scene the '
                                               'configuration names; earlier records of this benchmark ran it on '
                                               'spheres and boxes, the figure below')
      # the same net on the clouds of the earlier records (3 spheres + 2 boxes): fewer rows per level
      v = bench_unet.run(['--steps', '10', '--warmup', '5', '--fresh', '0', '--prefetch', '0', '--scene', 'mixed'])
      result['configs4_unet']['spheres_and_boxes'] = {k: v[k] for k in ('scene', 'ms_per_step', 'rows_per_depth')}
    except Exception as e:                              # supporting figure only
      result['configs4_unet'] = {'error': repr(e)}

  if extras and default_workload:
    # ---- the reference's own layer benchmark (test/benchmark_conv.py), bf16 (bench_sweep.py) ----
    try:
      import bench_sweep
      result['reference_benchmark_sweep'] = [
          {k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()}
          for r in bench_sweep.run([5, 6, 7, 8, 9, 10], ['bfloat16'])]
    except Exception as e:                              # supporting figure only
      result['reference_benchmark_sweep'] = {'error': repr(e)}

  if not args.no_cpu:
    result['cpu_baseline'] = cpu_baseline(torch, table, rows, C, C, args.cpu_rows)
    result['cpu_baseline']['octree'] = cpu_baseline_octree(pts, pc.normals.cpu(), bid if args.batch > 1 else None,
                                                           depth, args.batch)
  print(json.dumps(result))


if __name__ == '__main__':
  main()
