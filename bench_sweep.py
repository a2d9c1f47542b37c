"""The reference's own layer benchmark (test/benchmark_conv.py) on this library: one 3x3x3 stride-1
OctreeConv with bias on the non-empty nodes of a thin spherical shell, depth 5 .. 10 with 256, 128,
128, 64, 32, 32 channels, forward and backward timed apart (and both together replayed from a HIP
graph), fp32 / fp16 / bf16.  Prints one table
with the figures the reference publishes for its Triton kernels on an RTX 4090 beside ours
(test/benchmark/results.csv; other hardware, for orientation only) and one JSON line.

  python bench_sweep.py [--depths 5,6,7,8,9,10] [--dtypes float32,float16,bfloat16]
"""

import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path[:0] = [ROOT, os.path.join(ROOT, 'ocnn-pytorch_amd')]

CHANNELS = {5: 256, 6: 128, 7: 128, 8: 64, 9: 32, 10: 32}       # test/benchmark_conv.py:21
# ms of `OctConvT` (the Triton kernels) on an RTX 4090, test/benchmark/results.csv:18-23, 27-32,
# 36-41 (fwd) and :45-50, 54-59, 63-68 (bwd); fp32 ran with TF32 allowed
PUBLISHED = {
    'fwd': {'float32': [0.249, 0.226, 1.141, 0.787, 0.986, 3.972],
            'float16': [0.151, 0.136, 0.837, 0.428, 0.819, 3.067],
            'bfloat16': [0.151, 0.135, 0.831, 0.425, 0.786, 3.045]},
    'bwd': {'float32': [0.487, 0.497, 1.828, 1.954, 2.570, 10.326],
            'float16': [0.326, 0.318, 1.000, 1.224, 1.698, 7.584],
            'bfloat16': [0.323, 0.316, 0.996, 1.216, 1.690, 7.543]},
}


def timed(torch, fn, min_ms=25.0, reps=20):
  """Median-free mean over `reps` calls after at least `min_ms` of warm-up (the reference's
  triton.testing.do_bench warms up for 25 ms too)."""
  fn()
  torch.cuda.synchronize()
  s = torch.cuda.Event(enable_timing=True)
  e = torch.cuda.Event(enable_timing=True)
  s.record()
  fn()
  e.record()
  torch.cuda.synchronize()
  one = max(s.elapsed_time(e), 1e-3)
  for _ in range(int(min_ms / one) + 1):
    fn()
  torch.cuda.synchronize()
  s.record()
  for _ in range(reps):
    fn()
  e.record()
  torch.cuda.synchronize()
  return s.elapsed_time(e) / reps


def graph_replay_ms(torch, conv, x, octree, depth, gout):
  """Forward + backward of the layer captured once in a HIP graph (the library only launches
  kernels on the caller's stream), ms per replay: what is left when the host-side launch path
  is taken out.  No autograd graph of an earlier eager run may be alive: its gradient
  accumulation nodes belong to the stream they were made on, and a capture cannot wait for it."""
  params = [x] + list(conv.parameters())
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    for _ in range(2):
      for p in params:
        p.grad = None
      conv(x, octree, depth).backward(gout)
  torch.cuda.current_stream().wait_stream(side)
  torch.cuda.synchronize()
  for p in params:
    p.grad = None
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    conv(x, octree, depth).backward(gout)
  ms = timed(torch, graph.replay)
  del graph
  return ms


def run(depths, dtypes):
  """The records of the sweep: one per (depth, dtype)."""
  import torch
  from ocnn_amd import synthetic
  from ocnn_amd.nn import OctreeConv
  from ocnn_amd.octree import Octree, Points
  dev = 'cuda'
  records = []
  for depth in depths:
    c = CHANNELS[depth]
    octree = Octree(depth, 2)
    octree.build_octree(Points(synthetic.shell_points(depth, dev)))
    octree.construct_all_neigh()
    rows = int(octree.nnum_nempty[depth])
    nnz = int((octree._table(depth, '333', 1, True) >= 0).sum())
    for name in dtypes:
      dtype = getattr(torch, name)
      g = torch.Generator().manual_seed(depth)
      conv = OctreeConv(c, c, [3], 1, nempty=True, use_bias=True).to(dev).to(dtype)
      x = torch.randn(rows, c, generator=g).to(dtype).to(dev).requires_grad_()
      out = conv(x, octree, depth)
      gout = torch.randn(out.shape, generator=g).to(dtype).to(dev)
      if not records:
        # the first measurement of a process has now and then held a one-off pause of some 40 ms
        # (2 ms on the mean of 20 calls): one untimed round of the same calls first
        timed(torch, lambda: conv(x, octree, depth))
        timed(torch, lambda: out.backward(gout, retain_graph=True))
      fwd = timed(torch, lambda: conv(x, octree, depth))
      bwd = timed(torch, lambda: out.backward(gout, retain_graph=True))
      del out                 # with it the autograd graph of the eager runs and its nodes on this stream
      replay = graph_replay_ms(torch, conv, x.detach().clone().requires_grad_(), octree, depth, gout)
      i = depth - 5
      records.append({'depth': depth, 'channels': c, 'rows': rows, 'nnz': nnz, 'dtype': name,
                      'fwd_ms': fwd, 'bwd_ms': bwd, 'fwd_bwd_hip_graph_ms': replay,
                      'eff_tflops_fwd_bwd': 6.0 * nnz * c * c / (fwd + bwd) / 1e9,
                      'published_rtx4090_triton_fwd_ms': PUBLISHED['fwd'][name][i],
                      'published_rtx4090_triton_bwd_ms': PUBLISHED['bwd'][name][i]})
      del conv, x, gout
    del octree
    torch.cuda.empty_cache()
  return records


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--depths', default='5,6,7,8,9,10')
  ap.add_argument('--dtypes', default='float32,float16,bfloat16')
  ap.add_argument('--gpus', type=int, default=1)
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit('bench_sweep.py measures one GPU; --gpus %d is not supported' % args.gpus)
  records = run([int(d) for d in args.depths.split(',')], args.dtypes.split(','))
  print('%5s %4s %9s %-9s %8s %8s %10s %10s   %s' % ('depth', 'C', 'rows', 'dtype', 'fwd ms', 'bwd ms', 'TFLOP/s',
                                                   'graph ms', 'reference (Triton, RTX 4090) fwd / bwd ms'))
  for r in records:
    print('%5d %4d %9d %-9s %8.3f %8.3f %10.1f %10.3f   %.3f / %.3f' % (
        r['depth'], r['channels'], r['rows'], r['dtype'], r['fwd_ms'], r['bwd_ms'], r['eff_tflops_fwd_bwd'],
        r['fwd_bwd_hip_graph_ms'], r['published_rtx4090_triton_fwd_ms'], r['published_rtx4090_triton_bwd_ms']))
  print(json.dumps({'benchmark': 'test/benchmark_conv.py sweep, 3x3x3 stride 1, non-empty nodes, bias',
                    'data': 'synthetic (spherical shell of the reference benchmark)', 'n_gpus': 1,
                    'records': records}))


if __name__ == '__main__':
  main()
