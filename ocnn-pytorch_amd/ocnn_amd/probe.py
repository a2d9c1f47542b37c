"""ctypes binding of libocnn_probe.so: what the GPU itself sustains (MFMA rate with given
operand statistics, LDS read / write rate for a given address pattern).  Used by bench.py to
put the kernels' figures next to the part's; not part of the operator library."""

import ctypes
import os
from ctypes import c_double, c_int, c_void_p, POINTER, byref

import torch

from . import build as _build

_lib = None


def lib():
  global _lib
  if _lib is None:
    if not os.path.exists(_build.PROBE_LIB_PATH):
      _build.build_library()
    h = ctypes.CDLL(_build.PROBE_LIB_PATH)
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
  """The bf16 MFMA loop with two accumulator chains, alone (mix=False) or with the side work of
  the register-resident gather-GEMM kernel in its proportions (per 8 MFMAs: 16 VALU operations,
  six 16-byte LDS reads, one 16-byte write, two 2-byte reads).  Returns dict(tflops, ms,
  ticks_per_mfma, ns_per_mfma, ghz)."""
  g = torch.Generator().manual_seed(1)
  n = 9 * 256 * 8
  src = {'zero': torch.zeros(n), 'constant': torch.full((n,), 0.5),
         'uniform': torch.rand(n, generator=g) * 2 - 1, 'normal': torch.randn(n, generator=g)}[operands]
  src = src.to(torch.bfloat16).to(device)
  out = torch.empty(_cus(device) * 256, dtype=torch.float32, device=device)
  ticks = torch.zeros(_cus(device), dtype=torch.int64, device=device)
  ms, flops = c_double(), c_double()
  rc = lib().ocnn_probe_mfma_mix(int(bool(mix)), src.data_ptr(), out.data_ptr(), ticks.data_ptr(), iters,
                                 torch.cuda.current_stream().cuda_stream, byref(ms), byref(flops))
  if rc != 0:
    raise RuntimeError('ocnn_probe_mfma_mix failed')
  per = iters * 8
  t, ns = float(ticks.double().mean()) / per, ms.value * 1e6 / per
  return {'tflops': flops.value / ms.value / 1e9, 'ms': ms.value, 'ticks_per_mfma': t, 'ns_per_mfma': ns,
          'ghz': t / ns}


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
