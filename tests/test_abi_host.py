"""CPU checks of the shipped package: the C-ABI library loads and exports every
symbol the header declares, the host-evaluable kernel arithmetic agrees with
the oracle, and the host-side logic (shapes, errors, no CPU fallback)."""

import ctypes
import os
import re

import numpy as np
import pytest
import torch

import ocnn_amd
from ocnn_amd import _lib
from oracle import octree_ref as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
  text = open(os.path.join(ROOT, 'include', 'ocnn_hip.h')).read()
  text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
  return sorted(set(re.findall(r'\b(ocnn_[a-z0-9_]+)\s*\(', text)))


def _launching_entry_points():
  """Entry points that return a status and take a pointer: everything but the size queries, the
  *_supported / *_choose predicates and the host evaluations of kernel arithmetic."""
  names = set()
  for name, (res, args) in _lib.SIGNATURES.items():
    if res is ctypes.c_int and any(a is ctypes.c_void_p or hasattr(a, '_type_') and not isinstance(a._type_, str)
                                   for a in args):
      names.add(name)
  return names


def test_entry_points_refuse_bad_pointers_and_sizes_before_any_launch():
  """Every launching entry point, called with valid sizes, refuses a NULL in place of each array it
  reads or writes, a negative size and a missing workspace with an error code, before anything is
  launched.  The calls are made by a child process to which no GPU is visible, so an entry point
  that let one through would fail to launch there, not fault."""
  import json
  import subprocess
  import sys
  sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
  import abi_null_cases
  assert set(abi_null_cases.CASES) == _launching_entry_points()
  env = dict(os.environ, HIP_VISIBLE_DEVICES='-1', ROCR_VISIBLE_DEVICES='-1', CUDA_VISIBLE_DEVICES='-1')
  res = subprocess.run([sys.executable, os.path.join(ROOT, 'tests', 'abi_null_cases.py')], env=env,
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=600)
  assert res.returncode == 0, res.stderr[-2000:]
  got = json.loads(res.stdout.strip().splitlines()[-1])
  if 'skipped' in got:
    pytest.skip(got['skipped'])
  ERR_ARG, ERR_HIP, ERR_WS = -1, -2, -3
  for name, r in got.items():
    assert r['all_null'][0] == ERR_ARG, (name, r['all_null'])
    for i, (rc, msg) in r['one_null'].items():
      assert rc == ERR_ARG and 'null' in msg.lower(), (name, 'argument', i, rc, msg)
    for i, (rc, msg) in r['negative'].items():
      assert rc in (ERR_ARG, ERR_WS), (name, 'argument', i, rc, msg)
    if r['no_workspace'] is not None:
      assert r['no_workspace'][0] < 0, (name, r['no_workspace'])
    # the sizes of the case are valid: with every pointer set the call gets as far as the device
    assert r['good'][0] == (0 if name in abi_null_cases.HOST_ONLY else ERR_HIP), (name, r['good'])


def test_library_exports_every_declared_symbol():
  names = declared_symbols()
  assert len(names) >= 30
  handle = ctypes.CDLL(ocnn_amd.build.LIB_PATH)
  for name in names:
    assert hasattr(handle, name), name
  assert sorted(_lib.SIGNATURES) == names          # the binding covers the header exactly
  assert _lib.lib().ocnn_abi_version() == 1


@pytest.mark.parametrize('depth', [1, 4, 8, 9, 13, 16])
def test_host_key_arithmetic_matches_oracle(depth):
  L = _lib.lib()
  rng = np.random.default_rng(depth)
  xyz = rng.integers(-3, (1 << depth) + 3, size=(300, 3))
  b = rng.integers(0, 32768, size=300)
  want = R.xyz2key(xyz[:, 0], xyz[:, 1], xyz[:, 2], b, depth)
  buf = (ctypes.c_int64 * 4)()
  for i in range(300):
    got = L.ocnn_host_encode_key(int(xyz[i, 0]), int(xyz[i, 1]), int(xyz[i, 2]), int(b[i]), depth)
    assert got == int(want[i])
    L.ocnn_host_decode_key(got, depth, buf)
    x, y, z, bb = R.key2xyz(np.array([got]), depth)
    assert list(buf) == [int(x[0]), int(y[0]), int(z[0]), int(bb[0])]


def test_host_child_slot_lut_matches_reference_tables():
  L = _lib.lib()
  lut_parent, lut_child = R.neigh_luts()
  lp, lc = ctypes.c_int(), ctypes.c_int()
  for j in range(8):
    for k in range(27):
      L.ocnn_host_child_slot_lut(j, k, ctypes.byref(lp), ctypes.byref(lc))
      assert (lp.value, lc.value) == (int(lut_parent[j, k]), int(lut_child[j, k]))


def test_octree_public_luts_and_errors():
  o = ocnn_amd.Octree(depth=5, full_depth=2, batch_size=2)
  lut_parent, lut_child = R.neigh_luts()
  assert np.array_equal(o.lut_parent.numpy(), lut_parent)
  assert np.array_equal(o.lut_child.numpy(), lut_child)
  for k, v in R.LUT_KERNEL.items():
    assert o.lut_kernel[k].tolist() == v
  assert o.nnum.dtype == torch.long and o.nnum.device.type == 'cpu'
  assert len(o.neighs) == 6 and o.neighs[3] is None
  with pytest.raises(ValueError):
    o.get_neigh(3, '123')
  with pytest.raises(ValueError):
    o.get_neigh(3, '333', stride=3)


def test_neighbour_tables_need_a_full_first_layer():
  """The table of a layer below the full ones is made from its parents' table, and layer 0 has
  none: with full_depth = 0 the library refuses (an error code before any launch) instead of
  reading a table that does not exist; the reference's construct_neigh(1) fails there too."""
  L = _lib.lib()
  P = lambda *v: (ctypes.c_void_p * len(v))(*v)
  N = lambda *v: (ctypes.c_int64 * len(v))(*v)
  assert L.ocnn_neigh_all(2, 0, 1, N(1, 8, 64), N(1, 8, 64), P(None, None, None), P(None, None, None),
                          P(None, None, None), None) != 0
  assert 'full_depth' in L.ocnn_last_error().decode()
  assert L.ocnn_neigh_from_parent(None, None, None, 8, None, None, None) != 0
  assert 'null' in L.ocnn_last_error().decode()


def test_no_cpu_fallback():
  pts = ocnn_amd.Points(torch.rand(10, 3) * 0.5)
  o = ocnn_amd.Octree(depth=4, full_depth=2)
  with pytest.raises(RuntimeError):
    o.build_octree(pts)
  with pytest.raises(RuntimeError):
    ocnn_amd.octree.xyz2key(torch.zeros(3), torch.zeros(3), torch.zeros(3), depth=4)
  with pytest.raises(RuntimeError):
    o.construct_neigh(1)


def test_module_contract():
  from ocnn_amd.nn import OctreeConv, OctreeDeconv, OctreeDWConv
  c = OctreeConv(3, 5, [3], stride=1, nempty=True, use_bias=True)
  assert tuple(c.weights.shape) == (27, 3, 5) and tuple(c.bias.shape) == (5,)
  assert c.kernel == '333' and c.kernel_size == [3, 3, 3] and c.kdim == 27
  assert set(c.state_dict()) == {'weights', 'bias'}
  d = OctreeDeconv(3, 5, [2], stride=2)
  assert tuple(d.weights.shape) == (8, 5, 3) and d.bias is None
  w = OctreeDWConv(7, [3, 1, 1])
  assert tuple(w.weights.shape) == (3, 1, 7) and not hasattr(w, 'bias')
  bound = (3.0 ** 0.5) * (2.0 / (27 * 3 + 27 * 5)) ** 0.5
  assert float(c.weights.abs().max()) <= bound
  with pytest.raises(ValueError):
    OctreeConv(3, 5, method='nope')
  assert 'kernel_size=[3, 3, 3]' in repr(c)


def test_points_normalize_and_merge():
  from ocnn_amd.octree import Points, merge_points
  p = Points(torch.tensor([[-1.0, 0.0, 0.5]]))
  assert torch.equal(p.normalize(-1.0, 1.0, 64), torch.tensor([[0.0, 32.0, 48.0]]))
  m = merge_points([Points(torch.zeros(2, 3)), Points(torch.ones(3, 3))])
  assert m.batch_size == 2 and m.batch_id.view(-1).tolist() == [0, 0, 1, 1, 1]
  assert m.batch_id.dtype == torch.float32
  with pytest.raises(AssertionError):
    Points(torch.zeros(2, 2))


def test_pair_plan_lists_and_groups():
  """ocnn_pair_plan_lists (host only): the lists cover every (slot, row of a tile) once, heavy
  slots are cut by rows, at most 32 lists in four groups of at most 8 whose loads differ by
  no more than the largest list."""
  L = _lib.lib()
  rng = np.random.default_rng(3)
  for K in (1, 3, 8, 9, 27):
    for trial in range(20):
      counts = rng.integers(0, 1000, size=K).astype(np.int64)
      if trial % 3 == 0:
        counts[rng.integers(0, K)] = 15000                   # one dominant slot (the centre)
      c = (ctypes.c_int64 * K)(*counts.tolist())
      lists = (ctypes.c_int32 * 32)()
      loads = (ctypes.c_int64 * 32)()
      gb = (ctypes.c_int32 * 5)()
      nl = ctypes.c_int(0)
      assert L.ocnn_pair_plan_lists(K, ctypes.addressof(c), ctypes.addressof(lists), ctypes.addressof(loads),
                                    ctypes.addressof(gb), ctypes.addressof(nl)) == 0
      nl = nl.value
      assert K <= nl <= 32 and list(gb)[0] == 0 and list(gb)[4] == nl
      cover = np.zeros((K, 128), int)
      for v in list(lists)[:nl]:
        k, r0, r1 = v & 255, (v >> 8) & 255, ((v >> 16) & 255) + 1
        assert 0 <= k < K and 0 <= r0 < r1 <= 128 and (r1 - r0) % 32 == 0
        cover[k, r0:r1] += 1
      assert (cover == 1).all()
      loads = np.array(list(loads)[:nl])
      assert loads.sum() == counts.sum()
      sums = []
      for g in range(4):
        assert 0 <= gb[g + 1] - gb[g] <= 8
        sums.append(int(loads[gb[g]:gb[g + 1]].sum()))
      if nl <= 28:                                           # (room in every group)
        assert max(sums) - min(sums) <= loads.max()
      if counts.max() * 24 > counts.sum() and K < 27:
        assert nl > K                                        # the heavy slot was cut


def test_plan_history_is_bounded_and_clearable():
  from ocnn_amd.octree.octree import PlanHistory
  h = PlanHistory()
  for kind in range(PlanHistory.MAX_KINDS + 5):
    for j in range(PlanHistory.MAX_PLANS + 7):
      h.note((kind, 2), ((j, '333', 1, False), False), pairs=j % 2 == 0)
  assert len(h._kinds) == PlanHistory.MAX_KINDS
  assert (0, 2) not in h._kinds                          # the kinds used least recently are dropped
  last = h.requests((PlanHistory.MAX_KINDS + 4, 2))
  assert len(last) == PlanHistory.MAX_PLANS and ((0, '333', 1, False), False) not in last
  key = ((PlanHistory.MAX_PLANS + 6, '333', 1, False), False)
  assert last[key] is True
  h.note((PlanHistory.MAX_KINDS + 4, 2), key)            # a later plain request keeps the pair-plan wish
  assert h.requests((PlanHistory.MAX_KINDS + 4, 2))[key] is True
  h.clear()
  assert h.requests((PlanHistory.MAX_KINDS + 4, 2)) == {}


def test_kernel_selection_is_consistent_with_the_predicates():
  """ocnn_conv_gather_choose / ocnn_conv_wgrad_choose (host arithmetic only): every choice is
  a kernel whose *_supported() predicate takes the shape and whose entry point's row ranges
  hold; shapes past those ranges fall through to the plan-free kernels instead of failing."""
  from ocnn_amd import _lib
  L = _lib.lib()
  BF = 2
  lim = 0xfff00000
  for rows in (1000, 40000, 1 << 21, 17_000_000, 70_000_000):
    for K in (27, 8, 3, 1):
      for cin, cout in ((64, 64), (32, 32), (96, 96), (128, 128), (256, 256), (64, 128), (4, 32), (32, 10)):
        for occ, reuse in ((0.6, 9.0), (0.15, 4.0), (0.6, 1.2)):
          for umax in (200, 416, 500, 2000):
            k = L.ocnn_conv_gather_choose(BF, rows, rows, K, cin, cout, 0, 1, umax, rows * 2, occ, reuse)
            if k == _lib.GATHER_RW:
              assert L.ocnn_conv_gather_rw_supported(BF, rows, K, cin, cout, umax) and rows * K * 2 < lim
            elif k == _lib.GATHER_SPARSE:
              assert L.ocnn_conv_gather_sparse_supported(BF, rows, K, cin, cout, umax)
              assert rows * cout * 2 <= lim and occ <= 0.3 and rows >= 32768
            elif k == _lib.GATHER_WIDE:
              assert L.ocnn_conv_gather_wide_supported(BF, rows, K, cin, cout, umax) and (reuse >= 2 or K == 8)
            elif k == _lib.GATHER_PLANNED:
              assert L.ocnn_conv_gather_planned_supported(BF, rows, cin, cout) and reuse >= 2
            elif k == _lib.GATHER_ZERO_PADDED:
              assert rows >= 16384 and (cin % 32 or cout % 16)
            else:
              assert k == _lib.GATHER_PLAIN
            w = L.ocnn_conv_wgrad_choose(BF, rows, rows, K, cin, cout, 0, 1, umax, rows * 2, occ)
            if w == _lib.WGRAD_SPARSE:
              assert L.ocnn_conv_wgrad_sparse_supported(BF, rows, rows, K, cin, cout, umax) and rows * K * 2 < lim
            elif w == _lib.WGRAD_PLANNED:
              assert L.ocnn_conv_wgrad_planned_supported(BF, rows, rows, K, cin, cout, umax) and rows * K * 2 < lim
            elif w == _lib.WGRAD_ZERO_PADDED:
              assert rows >= 16384 and (cin % 32 or cout % 32)
            else:
              assert w == _lib.WGRAD_PLAIN
  # the benchmark layer and its neighbours take the kernels built for them
  assert L.ocnn_conv_gather_choose(BF, 1885272, 1885272, 27, 64, 64, 0, 1, 366, 3400000, 0.61, 9.0) == _lib.GATHER_RW
  assert L.ocnn_conv_wgrad_choose(BF, 1885272, 1885272, 27, 64, 64, 0, 1, 366, 3400000, 0.61) == _lib.WGRAD_PLANNED
  assert L.ocnn_conv_gather_choose(BF, 925113, 925113, 27, 96, 96, 0, 1, 300, 2000000, 0.145, 4.0) == _lib.GATHER_SPARSE
  assert L.ocnn_conv_gather_choose(BF, 211136, 211136, 27, 256, 256, 0, 1, 400, 500000, 0.74, 9.0) == _lib.GATHER_WIDE
  assert L.ocnn_conv_gather_choose(BF, 235659, 235659, 1, 512, 128, 1, 0, 0, 0, 1.0, 0.0) == _lib.GATHER_DENSE_RW
  assert L.ocnn_conv_gather_choose(BF, 1000, 1000, 27, 64, 64, 0, 0, 0, 0, 1.0, 0.0) == _lib.GATHER_PLAIN
  # 128 output channels on more rows than 32-bit offsets of the output reach: not the pair-plan kernel
  big = 17_000_000
  assert L.ocnn_conv_gather_choose(BF, big, big, 27, 128, 128, 0, 1, 300, big * 2, 0.15, 4.0) != _lib.GATHER_SPARSE


def test_a_stale_library_is_not_loaded(monkeypatch):
  """The built libraries carry the hash of their sources; when a source changes, the loader
  builds again instead of loading the old binary."""
  from ocnn_amd import _lib, build
  assert build.is_current()                       # the tree's libraries match the tree's sources
  calls = []
  monkeypatch.setattr(build, 'source_hash', lambda: 'something else')
  monkeypatch.setattr(build, 'build_library', lambda verbose=False: calls.append(1))
  monkeypatch.setattr(_lib, '_lib', None)
  assert not build.is_current()
  _lib.lib()
  assert calls == [1]
