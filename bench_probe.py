"""ctypes binding of libbench_probe.so (bench_probe.hip): what the GPU itself sustains (MFMA rate
with given operand statistics, LDS read / write rate for a given address pattern).  Used by
bench.py to put the kernels' figures next to the part's; not part of the operator library."""

import ctypes
import hashlib
import os
import subprocess
import sys
from ctypes import c_double, c_int, c_void_p, POINTER, byref

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(ROOT, 'bench_probe.hip')
LIB_PATH = os.path.join(ROOT, 'libbench_probe.so')
STAMP_PATH = LIB_PATH + '.sha256'

_lib = None


def _source_hash():
  with open(SOURCE, 'rb') as f:
    return hashlib.sha256(f.read()).hexdigest()


def is_current():
  try:
    with open(STAMP_PATH) as f:
      return os.path.exists(LIB_PATH) and f.read().strip() == _source_hash()
  except OSError:
    return False


def build_library(verbose=False):
  """Compiles the probes for gfx950 (the operator library's compiler and flags)."""
  sys.path.insert(0, os.path.join(ROOT, 'ocnn-pytorch_amd'))
  from ocnn_amd import build as b
  cmd = [b._hipcc()] + b.COMMON + ['-shared', SOURCE, '-o', LIB_PATH]
  res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  if res.returncode != 0:
    raise RuntimeError('command failed: {}\n{}'.format(' '.join(cmd), res.stdout))
  with open(STAMP_PATH, 'w') as f:
    f.write(_source_hash() + '\n')
  if verbose:
    print('built', LIB_PATH)
  return LIB_PATH


def lib():
  global _lib
  if _lib is None:
    if not is_current():
      build_library()
    h = ctypes.CDLL(LIB_PATH)
    h.ocnn_probe_mfma_rate.restype = c_int
    h.ocnn_probe_mfma_rate.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, POINTER(c_double),
                                       POINTER(c_double)]
    h.ocnn_probe_lds_rate.restype = c_int
    h.ocnn_probe_lds_rate.argtypes = [c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                      POINTER(c_double), POINTER(c_double)]
    h.ocnn_probe_mfma_mix.restype = c_int
    h.ocnn_probe_mfma_mix.argtypes = h.ocnn_probe_mfma_rate.argtypes
    _lib = h
  return _lib


def _cus(dev):
  return torch.cuda.get_device_properties(dev).multi_processor_count


def mfma_rate(dtype=torch.bfloat16, operands='normal', iters=20000, device='cuda'):
  """Sustained v_mfma_f32_32x32x16 rate of the whole GPU, one wave per SIMD, 14 accumulators
  per wave.  operands: 'zero', 'constant' (0.5), 'uniform' (-1 .. 1) or 'normal' (N(0, 1), what
  the benchmark feeds).  Returns dict(tflops, ms, ticks_per_mfma, ns_per_mfma)."""
  g = torch.Generator().manual_seed(1)
  n = 9 * 256 * 8
  src = {'zero': torch.zeros(n), 'constant': torch.full((n,), 0.5),
         'uniform': torch.rand(n, generator=g) * 2 - 1, 'normal': torch.randn(n, generator=g)}[operands]
  src = src.to(dtype).to(device)
  out = torch.empty(_cus(device) * 256, dtype=torch.float32, device=device)
  ticks = torch.zeros(_cus(device), dtype=torch.int64, device=device)
  ms, flops = c_double(), c_double()
  rc = lib().ocnn_probe_mfma_rate(int(dtype == torch.bfloat16), src.data_ptr(), out.data_ptr(), ticks.data_ptr(),
                                  iters, torch.cuda.current_stream().cuda_stream, byref(ms), byref(flops))
  if rc != 0:
    raise RuntimeError('ocnn_probe_mfma_rate failed')
  per = iters * 14
  return {'tflops': flops.value / ms.value / 1e9, 'ms': ms.value,
          'ticks_per_mfma': float(ticks.double().mean()) / per, 'ns_per_mfma': ms.value * 1e6 / per}


def mfma_mix(mix=True, operands='normal', iters=30000, device='cuda'):
  """The bf16 MFMA loop with two accumulator chains, alone (mix=False / 0), with the side work of
  the register-resident gather-GEMM kernel in its proportions (mix=True / 1; per 8 MFMAs: 16 VALU
  operations, six 16-byte LDS reads, one 16-byte write, two 2-byte reads), or with one of
  MIX_VARIANTS.  Returns dict(tflops, ms, ticks_per_mfma, ns_per_mfma, ghz)."""
  g = torch.Generator().manual_seed(1)
  n = 9 * 256 * 8
  src = {'zero': torch.zeros(n), 'constant': torch.full((n,), 0.5),
         'uniform': torch.rand(n, generator=g) * 2 - 1, 'normal': torch.randn(n, generator=g)}[operands]
  src = src.to(torch.bfloat16).to(device)
  out = torch.empty(_cus(device) * 256, dtype=torch.float32, device=device)
  ticks = torch.zeros(_cus(device), dtype=torch.int64, device=device)
  ms, flops = c_double(), c_double()
  rc = lib().ocnn_probe_mfma_mix(int(mix), src.data_ptr(), out.data_ptr(), ticks.data_ptr(), iters,
                                 torch.cuda.current_stream().cuda_stream, byref(ms), byref(flops))
  if rc != 0:
    raise RuntimeError('ocnn_probe_mfma_mix failed')
  per = iters * 8
  t, ns = float(ticks.double().mean()) / per, ms.value * 1e6 / per
  return {'tflops': flops.value / ms.value / 1e9, 'ms': ms.value, 'ticks_per_mfma': t, 'ns_per_mfma': ns,
          'ghz': t / ns}


# side work per 8 MFMAs, by the variant number of ocnn_probe_mfma_mix
MIX_VARIANTS = [
    (0, 'no side work'),
    (2, '16 VALU'),
    (3, '32 VALU'),
    (4, '4 ds_read_b128'),
    (5, '6 ds_read_b128'),
    (6, '8 ds_read_b128'),
    (7, '8 ds_read_b128, two lanes per bank group'),
    (8, '1 ds_write_b128'),
    (9, '2 ds_write_b128'),
    (10, '2 ds_read_u16'),
    (1, 'the gather-GEMM kernel\'s: 16 VALU, 6 ds_read_b128, 1 ds_write_b128, 2 ds_read_u16'),
    (11, 'the same, two lanes per bank group'),
    (12, 'the same without the write'),
    (13, 'a wave that owns its outputs: 16 VALU, 8 ds_read_b128, 2 ds_read_u16'),
    (14, 'the kernel\'s with an s_barrier every 32 MFMAs'),
]


def lds_rate(offsets, write=False, iters=4000, device='cuda'):
  """offsets: int tensor (8, threads) of byte offsets into 64 KiB (multiples of 16), threads 256
  or 512 = one workgroup per CU.  Returns dict(tbytes_per_s, bytes_per_tick_per_cu, ms)."""
  threads = offsets.shape[1]
  addr = offsets.to(torch.int32).contiguous().to(device)
  n_cu = _cus(device)
  out = torch.empty(n_cu * threads, dtype=torch.float32, device=device)
  ticks = torch.zeros(n_cu, dtype=torch.int64, device=device)
  ms, nbytes = c_double(), c_double()
  rc = lib().ocnn_probe_lds_rate(int(write), threads, addr.data_ptr(), out.data_ptr(), ticks.data_ptr(), iters,
                                 torch.cuda.current_stream().cuda_stream, byref(ms), byref(nbytes))
  if rc != 0:
    raise RuntimeError('ocnn_probe_lds_rate failed')
  return {'tbytes_per_s': nbytes.value / ms.value / 1e9, 'ms': ms.value,
          'bytes_per_tick_per_cu': nbytes.value / n_cu / float(ticks.double().mean())}


def _gather_pattern(threads, rows_of_lane, seed=0):
  """Offsets of the gather-GEMM kernel's B-operand reads: lane (r32, q) of wave w reads the
  16-byte chunk 4 (w % 2) + q of LDS row p = rows_of_lane(j, r32, generator), stored at chunk
  c ^ ((p >> 1) & 7) of the 128-byte row."""
  g = torch.Generator().manual_seed(seed)
  out = torch.zeros(8, threads, dtype=torch.long)
  for t in range(threads):
    w, lane = t // 64, t % 64
    c0 = 4 * (w & 1) + (lane >> 5)
    for j in range(8):
      p = rows_of_lane(j, lane & 31, g)
      out[j, t] = p * 128 + ((c0 ^ (p >> 1)) & 7) * 16
  return out % 65536


def main():
  """Prints the tables kept under profiles/: MFMA rates by operand statistics, the MFMA loop
  with the gather-GEMM kernel's side work, LDS rates by address pattern."""
  torch.cuda.set_device(0)
  print('device:', torch.cuda.get_device_name(0), ' CUs:', _cus('cuda'))
  print('\nv_mfma_f32_32x32x16, one wave per SIMD, 14 accumulators per wave, all CUs:')
  for dt in (torch.bfloat16, torch.float16):
    for ops in ('zero', 'constant', 'uniform', 'normal'):
      r = mfma_rate(dt, ops, 20000)
      print('  %-9s operands %-9s %7.1f TFLOP/s  %5.2f ticks/MFMA  %5.2f ns/MFMA  (%.2f GHz)' % (
          str(dt)[6:], ops, r['tflops'], r['ticks_per_mfma'], r['ns_per_mfma'], r['ticks_per_mfma'] / r['ns_per_mfma']))
  print('\nbf16 MFMA loop, two accumulator chains, N(0,1) operands:')
  print('  (side work per 8 MFMAs of a wave)')
  for mix, name in MIX_VARIANTS:
    r = mfma_mix(mix, iters=20000)
    print('  %7.1f TFLOP/s  %5.2f ticks/MFMA  %5.2f ns/MFMA  (%.2f GHz)  %s' % (
        r['tflops'], r['ticks_per_mfma'], r['ns_per_mfma'], r['ghz'], name))
  print('\nLDS, 16 bytes per lane and access, one workgroup of 256 threads per CU (B / tick / CU):')
  lanes = torch.arange(256)
  patterns = [
      ('consecutive 16-byte chunks', torch.stack([(lanes % 64) * 16 + j * 1024 + (lanes // 64) * 8192 for j in range(8)])),
      ('stride 32 B (2 lanes per 16-bank group)', torch.stack([((lanes % 64) * 32 + j * 2048) % 65536 for j in range(8)])),
      ('stride 64 B', torch.stack([((lanes % 64) * 64 + j * 4096) % 65536 for j in range(8)])),
      ('stride 128 B (same chunk of consecutive rows, no swizzle)', torch.stack([((lanes % 64) * 128 + j * 8192) % 65536 for j in range(8)])),
      ('stride 256 B (all lanes on one bank group)', torch.stack([((lanes % 64) * 256) % 65536 for j in range(8)])),
      ('gathered rows: 32 consecutive rows per access, swizzled', _gather_pattern(256, lambda j, r, g: 1 + r + 32 * j)),
      ('gathered rows: two sibling groups 16 rows apart, swizzled', _gather_pattern(256, lambda j, r, g: 1 + (r % 8) + 16 * (r // 8) + 64 * j)),
      ('gathered rows: random rows 0..416, swizzled', _gather_pattern(256, lambda j, r, g: int(torch.randint(0, 417, (1,), generator=g)))),
  ]
  for name, off in patterns:
    rd, wr = lds_rate(off, False, 4000), lds_rate(off, True, 4000)
    print('  %-60s read %6.1f   write %6.1f   (read %.1f TB/s whole GPU)' % (
        name, rd['bytes_per_tick_per_cu'], wr['bytes_per_tick_per_cu'], rd['tbytes_per_s']))


if __name__ == '__main__':
  main()
