"""The entry point that allocates nothing (ocnn_conv_gather_rw_static) against the entry
point it is a variant of (ocnn_conv_gather_rw), through the C ABI: identical bits, on two
calls in a row of which the second has the smaller input, then on a 32 -> 32 layer; a layer
whose weights exceed the built-in buffer is rejected."""

import sys

import pytest
import torch

from ocnn_amd import _lib
from ocnn_amd.octree.octree import TilePlan

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


def _local_table(rows, rows_in, K, g, spread=40, empty=0.3):
  base = (torch.arange(rows, dtype=torch.float64) * (rows_in / max(rows, 1))).long()[:, None]
  off = torch.randint(-spread, spread + 1, (rows, K), generator=g)
  t = (base + off).clamp_(0, rows_in - 1).to(torch.int32)
  t[torch.rand(rows, K, generator=g) < empty] = -1
  return t


def _both(dtype, rows, rows_in, K, ch, g, transposed, reverse, with_bias):
  L = _lib.lib()
  table = _local_table(rows, rows_in, K, g).to(DEV)
  plan = TilePlan(table)
  x = torch.randn(rows_in, ch, generator=g).to(dtype).to(DEV)
  w = (torch.randn(K, ch, ch, generator=g) / (K * ch) ** 0.5).to(dtype).to(DEV)
  b = torch.randn(ch, generator=g).to(dtype).to(DEV) if with_bias else None
  code = _lib.dtype_code(x)
  assert L.ocnn_conv_gather_rw_supported(code, rows_in, K, ch, ch, plan.umax)
  ws = _lib.workspace(L.ocnn_conv_gather_workspace_bytes(code, rows_in, K, ch, ch), DEV)
  want = torch.full((rows, ch), float('nan'), dtype=dtype, device=DEV)
  got = torch.full((rows, ch), float('nan'), dtype=dtype, device=DEV)
  torch.cuda.synchronize()
  _lib.check(L.ocnn_conv_gather_rw(
      code, _lib.ptr(x), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax,
      plan.total, rows, K, _lib.ptr(w), ch, ch, int(transposed), int(reverse), _lib.ptr(b), _lib.ptr(want),
      _lib.ptr(ws), ws.numel(), _lib.stream()))
  # everything the second entry point touches exists by now: it may not allocate
  before = torch.cuda.memory_allocated()
  free_before = torch.cuda.mem_get_info()[0]             # hipMemGetInfo: sees a hipMalloc inside the library too
  _lib.check(L.ocnn_conv_gather_rw_static(
      code, _lib.ptr(x), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax,
      plan.total, rows, K, _lib.ptr(w), ch, ch, int(transposed), int(reverse), _lib.ptr(b), _lib.ptr(got),
      _lib.stream()))
  torch.cuda.synchronize()
  assert torch.cuda.memory_allocated() == before
  assert torch.cuda.mem_get_info()[0] >= free_before
  assert torch.isfinite(want.float()).all()
  assert torch.equal(got, want)


def test_static_entry_point_matches_the_workspace_one():
  L = _lib.lib()
  assert L.ocnn_conv_gather_rw_static_max_weight_bytes() == 27 * 64 * 64 * 2
  g = torch.Generator().manual_seed(77)
  say('no-alloc gather: 64 -> 64, K 27, 40001 rows')
  _both(torch.bfloat16, 40001, 39000, 27, 64, g, False, False, True)
  say('no-alloc gather: second call, smaller input (64 -> 64, K 9, 1000 rows)')
  _both(torch.bfloat16, 1000, 700, 9, 64, g, True, True, False)
  say('no-alloc gather: 32 -> 32, K 27, f16')
  _both(torch.float16, 5000, 5000, 27, 32, g, False, False, True)
  say('no-alloc gather: 64 -> 64 again after the smaller layers')
  _both(torch.float16, 12800, 12800, 27, 64, g, True, True, True)


def test_static_entry_point_rejects_what_it_cannot_hold():
  L = _lib.lib()
  x = torch.zeros(128, 128, dtype=torch.bfloat16, device=DEV)
  rc = L.ocnn_conv_gather_rw_static(2, _lib.ptr(x), 128, None, None, None, 0, 0, 128, 27, _lib.ptr(x), 128, 128, 0,
                                    0, None, _lib.ptr(x), _lib.stream())
  assert rc != 0
  assert b'not supported' in L.ocnn_last_error()
