"""What bench.py and bench_layers.py share: timing of one layer's forward + backward through its
module, and the algorithmic work (flops over non-empty neighbours, bytes with every tensor moved
once and 4-byte table entries) that the rates are quoted against."""

import time

PEAK_MFMA_16BIT_TFLOPS = 2500.0     # MI355X dense bf16 / fp16
PEAK_HBM_GBS = 8000.0


def build_octree(torch, synthetic, Octree, Points, cloud, batch, seed, n, depth, dev, repeats=3):
  """Builds the octree of `batch` synthetic clouds `repeats` times; returns the last octree, the
  best build and neighbour-table times in ms, the points and their batch ids."""
  pts, nrm, bid = synthetic.batch_clouds(cloud, batch, seed, n=n)
  pc = Points(pts.to(dev), nrm.to(dev), batch_id=bid.to(dev) if batch > 1 else None, batch_size=batch)
  times = []
  for _ in range(repeats):
    o = Octree(depth, 2, batch_size=batch)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    o.build_octree(pc)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    o.construct_all_neigh()
    torch.cuda.synchronize()
    times.append((t1 - t0, time.perf_counter() - t1))
  return o, min(t[0] for t in times) * 1e3, min(t[1] for t in times) * 1e3, pts, bid, pc


def layer_work(rows_in, table_rows, K, nnz, cin, cout, dw=False, es=2):
  """(flops, bytes) of forward + data gradient + weight gradient of one layer."""
  if dw:
    flops = 6.0 * nnz * cin
    nbytes = 3 * (es * (rows_in * cin + table_rows * cin + K * cin) + 4 * table_rows * K)
  else:
    flops = 6.0 * nnz * cin * cout
    nbytes = (3 * (es * (rows_in * cin + table_rows * cout) + 4 * table_rows * K) + 2 * es * K * cin * cout +
              4 * K * cin * cout)
  return flops, nbytes


def time_layer(torch, tag, mod, octree, depth, rows_in, cin, cout, table, dtype, steps, warmup, dev, dw=False):
  """Forward + backward of `mod` through autograd, `steps` times between events on the current
  stream; one record with ms, effective TFLOP/s and the fractions of the two roofs."""
  g = torch.Generator().manual_seed(7)
  mod = mod.to(dev).to(dtype)
  x = torch.randn(rows_in, cin, generator=g).to(dtype).to(dev).requires_grad_()
  out = mod(x, octree, depth)
  gout = torch.randn(out.shape, generator=g).to(dtype).to(dev)

  def step():
    x.grad = None
    mod.weights.grad = None
    mod(x, octree, depth).backward(gout)

  for _ in range(warmup):
    step()
  torch.cuda.synchronize()
  s = torch.cuda.Event(enable_timing=True)
  e = torch.cuda.Event(enable_timing=True)
  s.record()
  for _ in range(steps):
    step()
  e.record()
  torch.cuda.synchronize()
  ms = s.elapsed_time(e) / steps
  rows, K = table.shape
  nnz = int((table >= 0).sum())
  flops, nbytes = layer_work(rows_in, rows, K, nnz, cin, cout, dw)
  return {
      'layer': tag, 'dtype': str(dtype).replace('torch.', ''), 'rows_in': rows_in, 'rows_table': rows,
      'K': K, 'nnz': nnz, 'ms_fwd_bwd': ms, 'eff_tflops': flops / ms / 1e9,
      'frac_mfma_peak': flops / ms / 1e9 / PEAK_MFMA_16BIT_TFLOPS,
      'algorithmic_bytes': nbytes, 'frac_hbm_peak_at_algorithmic_bytes': nbytes / ms / 1e6 / PEAK_HBM_GBS,
  }
