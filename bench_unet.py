"""Forward + backward of the reference's segmentation U-Net (ocnn/models/unet.py:16-105: encoder
channels 32-32-64-128-256 with 2/3/4/6 residual blocks, decoder 256-256-128-96-96 with 2 each,
2x2x2 stride-2 (de)convolutions between levels, trilinear interpolation of the last features at
the query points, a 1x1 head) as this package assembles it (ocnn_amd/unet.py), on one MI355X.  Supporting data for the pieces around the convolutions (the headline number is
bench.py's): synthetic batch of 8 clouds x 150 000 points at depth 9 (indoor-like scenes: a floor,
walls and 10 - 20 boxes each; --scene mixed: 3 spheres and 2 boxes), input signal 'ND'
(normals + displacement), 10 classes, random weights, cross-entropy against random labels.

One JSON line: ms per forward + backward, and the share of the step spent in each kind of
kernel when --profile is given (torch profiler, device time).  ms_per_step is the step on a
resident octree; ms_octree_build_and_tables + ms_first_step_on_a_fresh_octree is what a step costs
when every batch brings a new octree (the plans of its tables are built inside that step);
ms_per_step_new_octree_built_on_a_side_stream is the step of a loop that builds the next octree and
its plans on a second stream while the device runs the step before (Octree.prepare).
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


def run(argv=None):
  """Runs the benchmark with the given command-line arguments (None: the process's) and returns
  the record that main() prints."""
  ap = argparse.ArgumentParser()
  ap.add_argument('--steps', type=int, default=10)
  ap.add_argument('--warmup', type=int, default=3)
  ap.add_argument('--batch', type=int, default=8)
  ap.add_argument('--points', type=int, default=150000)
  ap.add_argument('--depth', type=int, default=9)
  ap.add_argument('--dtype', default='bfloat16')
  ap.add_argument('--nempty', type=int, default=1)
  ap.add_argument('--profile', action='store_true')
  ap.add_argument('--fresh', type=int, default=3, help='steps on a newly built octree, timed after the others')
  ap.add_argument('--prefetch', type=int, default=6,
                  help='steps that each run on a new octree built (with its plans) on a side stream while '
                       'the step before is running')
  ap.add_argument('--scene', default='indoor', choices=['indoor', 'mixed'],
                  help='indoor: floor, walls and 10 - 20 boxes per cloud (the configuration\'s scene); '
                       'mixed: 3 spheres and 2 boxes')
  ap.add_argument('--torch-loss', action='store_true', help='torch.nn.functional.cross_entropy for the loss')
  args = ap.parse_args(argv)
  import torch
  from ocnn_amd import synthetic
  from ocnn_amd.unet import UNet
  from ocnn_amd.octree import Octree, Points
  assert torch.cuda.is_available(), 'bench_unet.py needs a GPU'
  dev = 'cuda:0'
  torch.cuda.set_device(0)
  dtype = getattr(torch, args.dtype)
  nempty = bool(args.nempty)

  maker = synthetic.indoor_cloud if args.scene == 'indoor' else synthetic.mixed_cloud
  pts, nrm, bid = synthetic.batch_clouds(maker, args.batch, 1004, n=args.points)
  pc = Points(pts.to(dev), nrm.to(dev), batch_id=bid.to(dev), batch_size=args.batch)
  def build():
    o = Octree(args.depth, 2, batch_size=args.batch)
    o.build_octree(pc)
    o.construct_all_neigh()
    return o

  octree = build()
  feat = octree.get_input_feature('ND', nempty).to(dtype)
  query = torch.cat([pts.to(dev), bid.to(dev).float().view(-1, 1)], 1)     # xyz in [-1, 1], batch index
  labels = torch.randint(0, 10, (query.shape[0],), generator=torch.Generator().manual_seed(5)).to(dev)
  torch.manual_seed(0)
  net = UNet(feat.shape[1], 10, 'linear', nempty).to(dev).to(dtype)
  params = [p for p in net.parameters()]

  def step(octree=octree):
    for p in params:
      p.grad = None
    logits = net(feat, octree, args.depth, query.clone())   # (the interpolation rescales its points in place)
    if args.torch_loss:
      loss = torch.nn.functional.cross_entropy(logits.float(), labels)
    else:
      # the same cross-entropy; torch's nll_loss kernels take 1.7 ms on 1.2 M x 10 logits
      lf = logits.float()
      loss = (torch.logsumexp(lf, 1) - lf.gather(1, labels.view(-1, 1)).squeeze(1)).mean()
    loss.backward()

  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  t0 = time.perf_counter()
  for _ in range(args.steps):
    step()
  torch.cuda.synchronize()
  ms = (time.perf_counter() - t0) / args.steps * 1e3
  # a training loop sees a new octree every step: build, tables, plans and the step on it
  fresh = []
  for _ in range(args.fresh):
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    o = build()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    step(o)
    torch.cuda.synchronize()
    fresh.append(((t1 - t0) * 1e3, (time.perf_counter() - t1) * 1e3))
  fresh.sort(key=lambda v: v[0] + v[1])
  mid = fresh[len(fresh) // 2] if fresh else (None, None)
  # the same with the next octree built ahead: the host has queued the whole step long before the
  # device is through with it, so the build of the next octree, on a stream of its own, runs
  # beside the step's kernels (its read-backs wait for that stream only)
  ms_prefetch = None
  if args.prefetch > 0:
    side, main = torch.cuda.Stream(), torch.cuda.current_stream()
    torch.cuda.synchronize()                      # (the points are on the device by now: the side stream need not wait for main's queue)

    def ahead():
      with torch.cuda.stream(side):
        o = build().prepare()
        f = o.get_input_feature('ND', nempty).to(dtype)
      return o, f

    def prefetch_steps(n, nxt):
      nonlocal feat
      for _ in range(n):
        main.wait_stream(side)
        o, feat = nxt
        o.record_stream(main)
        feat.record_stream(main)
        step(o)
        nxt = ahead()
      torch.cuda.synchronize()
      return nxt

    nxt = prefetch_steps(2, ahead())
    t0 = time.perf_counter()
    prefetch_steps(args.prefetch, nxt)
    ms_prefetch = (time.perf_counter() - t0) / args.prefetch * 1e3
    feat = octree.get_input_feature('ND', nempty).to(dtype)
  out = {'net': 'U-Net (ocnn/models/unet.py), forward + backward', 'ms_per_step': ms,
         'ms_octree_build_and_tables': mid[0], 'ms_first_step_on_a_fresh_octree': mid[1],
         'ms_per_step_new_octree_built_on_a_side_stream': ms_prefetch,
         'dtype': args.dtype, 'scene': args.scene,
         'nempty': nempty, 'batch': args.batch, 'points': int(pts.shape[0]), 'depth': args.depth,
         'rows_per_depth': (octree.nnum_nempty if nempty else octree.nnum).tolist(),
         'parameters': sum(p.numel() for p in params)}
  if args.profile:
    from torch.profiler import profile, ProfilerActivity
    with profile(activities=[ProfilerActivity.CUDA, ProfilerActivity.CPU]) as prof:
      step()
      torch.cuda.synchronize()
    groups, top = {}, []
    for e in prof.key_averages():
      t = getattr(e, 'device_time_total', 0) or getattr(e, 'cuda_time_total', 0)
      name = e.key
      if t <= 0 or not any(k in name for k in ('ocnn', 'Kernel', 'kernel', 'Cijk', 'gemm')):
        continue
      if 'conv_' in name or 'wgrad' in name or 'pack_weights' in name:
        k = 'octree conv kernels'
      elif 'batch_norm' in name or 'BatchNorm' in name or 'bn_' in name:
        k = 'batch norm'
      elif 'interp' in name or 'csr_rows' in name or 'search' in name:
        k = 'interpolation'
      elif 'pad' in name and 'ocnn' in name:
        k = 'pad / depad'
      elif 'tile_plan' in name or 'neigh' in name:
        k = 'tables / plans'
      elif 'Cijk' in name or 'gemm' in name:
        k = 'dense GEMM (1x1)'
      else:
        k = 'elementwise / other'
      groups[k] = groups.get(k, 0.0) + t / 1e3
      top.append((round(t / 1e3, 3), e.count, name[:90]))
    out['device_ms_by_kind'] = {k: round(v, 3) for k, v in sorted(groups.items(), key=lambda kv: -kv[1])}
    out['top_kernels_ms_calls'] = sorted(top, reverse=True)[:24]
  return out


def main():
  print(json.dumps(run()), flush=True)


if __name__ == '__main__':
  main()
