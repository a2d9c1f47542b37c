"""Octree construction, neighbour search and tile plan on their own: the clouds of configs[1]
(8 x 100 k points, depth 8) and configs[3] (4 x 250 k points, depth 9) built `--steps` times, one
JSON line per configuration with the time of each stage and the neighbour tables' bytes against
the HBM peak.  The program the rocprofv3 summaries of these kernels under profiles/ run.

  python bench_octree.py [--steps 10] [--configs 1,3]
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [ROOT, os.path.join(ROOT, 'ocnn-pytorch_amd')]

from bench_common import PEAK_HBM_GBS   # noqa: E402


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--steps', type=int, default=10)
  ap.add_argument('--configs', default='1,3')
  ap.add_argument('--gpus', type=int, default=1)
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit('bench_octree.py measures one GPU; --gpus %d is not supported' % args.gpus)
  import torch
  from ocnn_amd import synthetic
  from ocnn_amd.octree import Octree, Points
  from ocnn_amd.octree.octree import TilePlan
  dev = 'cuda'
  shapes = {'1': (synthetic.mixed_cloud, 8, 1001, 100000, 8), '3': (synthetic.planes_cloud, 4, 1003, 250000, 9)}
  for name in args.configs.split(','):
    cloud, batch, seed, n, depth = shapes[name]
    pts, nrm, bid = synthetic.batch_clouds(cloud, batch, seed, n=n)
    pc = Points(pts.to(dev), nrm.to(dev), batch_id=bid.to(dev), batch_size=batch)
    stages = {'build_octree': [], 'construct_all_neigh': [], 'tile_plan_333': []}
    for it in range(args.steps + 2):
      o = Octree(depth, 2, batch_size=batch)
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      o.build_octree(pc)
      torch.cuda.synchronize()
      t1 = time.perf_counter()
      o.construct_all_neigh()
      torch.cuda.synchronize()
      t2 = time.perf_counter()
      table = o._table(depth, '333', 1, False)
      torch.cuda.synchronize()
      t3 = time.perf_counter()
      TilePlan(table)
      torch.cuda.synchronize()
      t4 = time.perf_counter()
      if it >= 2:                                      # two warm-up builds
        for key, dt in zip(stages, (t1 - t0, t2 - t1, t4 - t3)):
          stages[key].append(dt * 1e3)
    ms = {k: statistics.median(v) for k, v in stages.items()}
    neigh_bytes = sum(int(o.nnum[d]) * 27 * 4 + int(o.nnum_nempty[d - 1]) * 27 * 4 + int(o.nnum[d - 1]) * 4
                      for d in range(1, depth + 1))
    plan_bytes = int(o.nnum[depth]) * 27 * (4 + 2)      # the table read, 16-bit positions written
    print(json.dumps({
        'octree': 'configs[%s]: batch %d x %d points, depth %d' % (name, batch, n, depth),
        'points': int(pts.shape[0]), 'nnum': o.nnum.tolist(), 'nnum_nempty': o.nnum_nempty.tolist(),
        'build_octree_ms': ms['build_octree'], 'construct_all_neigh_ms': ms['construct_all_neigh'],
        'tile_plan_ms': ms['tile_plan_333'], 'steps': args.steps,
        'construct_all_neigh_algorithmic_bytes': neigh_bytes,
        'construct_all_neigh_frac_hbm_peak': neigh_bytes / ms['construct_all_neigh'] / 1e6 / PEAK_HBM_GBS,
        'tile_plan_algorithmic_bytes': plan_bytes,
        'tile_plan_frac_hbm_peak': plan_bytes / ms['tile_plan_333'] / 1e6 / PEAK_HBM_GBS,
        'build_octree_mpoints_per_s': pts.shape[0] / ms['build_octree'] / 1e3,
    }), flush=True)


if __name__ == '__main__':
  main()
