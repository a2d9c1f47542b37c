"""The layers on an octree that is NOT this package's class: an object holding only what the
reference's layers read of an octree (ocnn/nn/octree_conv.py:51-100: `get_neigh`, `children`,
`nnum`, `nnum_nempty`), filled from the arrays of the reference's own fixture batch_45.npz.
OctreeConv / OctreeDeconv / OctreeDWConv run on it and match the fp64 oracle on the same arrays.
"""

import os
import sys

import numpy as np
import pytest
import torch

from ocnn_amd.nn import OctreeConv, OctreeDeconv, OctreeDWConv, octree_depad, octree_pad
from ocnn_amd.octree import ContractOctree, Octree, tables_of
from oracle import conv_ref as C
from oracle import octree_ref as R

pytestmark = pytest.mark.gpu
DEV = 'cuda'
TOL = {torch.float32: 1e-4, torch.float16: 2e-2, torch.bfloat16: 2e-2}

COLUMNS = {'333': list(range(27)), '222': [13, 14, 16, 17, 22, 23, 25, 26], '311': [4, 13, 22], '131': [10, 13, 16],
           '113': [12, 13, 14], '331': [1, 4, 7, 10, 13, 16, 19, 22, 25], '313': [3, 4, 5, 12, 13, 14, 21, 22, 23],
           '133': [9, 10, 11, 12, 13, 14, 15, 16, 17]}


def say(*a):
  print(*a, flush=True)
  sys.stdout.flush()


class BareOctree:
  """What a layer of the reference reads of an octree, as tensors on `device`, and nothing
  else: no tables cache, no plans, none of this package's private members."""

  def __init__(self, d, device, child_dtype=torch.int32):
    self.depth, self.full_depth = int(d['depth']), int(d['full_depth'])
    nnum = [int(v) for v in d['nnum']]
    self.nnum = torch.tensor(nnum, dtype=torch.long)
    self.nnum_nempty = torch.tensor([int(v) for v in d['nnum_nempty']], dtype=torch.long)
    ends = np.cumsum(nnum)
    self.children = [torch.from_numpy(d['child'][e - n:e].copy()).to(child_dtype).to(device) for n, e in zip(nnum, ends)]
    # the fixture holds the tables of depths 1 .. depth, one after the other
    self.neighs = [None] + [torch.from_numpy(d['neigh'][e - n - nnum[0]:e - nnum[0]].astype(np.int64)).to(device)
                            for n, e in zip(nnum[1:], ends[1:])]

  def get_neigh(self, depth, kernel='333', stride=1, nempty=False):
    """Rows: all nodes, every eighth (stride 2) or the non-empty ones; entries renumbered among
    the non-empty nodes with nempty; columns by kernel (ocnn/octree/octree.py:490-523)."""
    table = self.neighs[depth]
    child = self.children[depth].long()
    if stride == 2:
      table = table[::8]
    elif nempty:
      table = table[child >= 0]
    if nempty:
      table = torch.where(table >= 0, child[table.clamp_min(0)], table)
    return table[:, COLUMNS[kernel]].contiguous()


def reference_octree(d):
  """The same arrays in the oracle's container."""
  ref = R.OctreeRef(int(d['depth']), int(d['full_depth']), 2)
  nnum = [int(v) for v in d['nnum']]
  ends = np.cumsum(nnum)
  for depth, (n, e) in enumerate(zip(nnum, ends)):
    ref.children[depth] = d['child'][e - n:e].astype(np.int32)
    if depth >= 1:
      ref.neighs[depth] = d['neigh'][e - n - nnum[0]:e - nnum[0]].astype(np.int64)
  ref.nnum[:] = nnum
  ref.nnum_nempty[:] = d['nnum_nempty']
  return ref


@pytest.fixture(scope='module')
def fixture(ref_data):
  d = np.load(os.path.join(ref_data, 'batch_45.npz'))
  return d, reference_octree(d)


def f64(t):
  return t.detach().double().cpu().numpy()


def rel_err(got, want):
  return float(np.abs(f64(got) - want).max()) / max(1e-30, float(np.abs(want).max()))


def run(kind, octree, ref, depth, ks, stride, nempty, cin, cout, dtype, seed):
  g = torch.Generator().manual_seed(seed)
  ks3 = (list(ks) + [ks[-1]] * 3)[:3]
  K = ks3[0] * ks3[1] * ks3[2]
  if kind == 'conv':
    mod, layer = OctreeConv(cin, cout, ks, stride, nempty, use_bias=True), C.conv_layer
  elif kind == 'deconv':
    mod, layer = OctreeDeconv(cin, cout, ks, stride, nempty, use_bias=True), C.deconv_layer
  else:
    mod, layer = OctreeDWConv(cin, ks, stride, nempty, use_bias=True), C.dwconv_layer
  with torch.no_grad():
    mod.weights.copy_(torch.randn(mod.weights.shape, generator=g) / (K * cin) ** 0.5)
    mod.bias.copy_(torch.randn(mod.bias.shape, generator=g))
  mod = mod.to(DEV).to(dtype)
  in_rows = ref.nnum_nempty[depth] if nempty or (kind == 'deconv' and stride == 2) else ref.nnum[depth]
  if kind == 'deconv' and stride == 2 and not nempty:
    in_rows = ref.nnum[depth]                              # the module depads its input itself
  data = torch.randn(int(in_rows), cin, generator=g).to(dtype)
  x = data.to(DEV).requires_grad_()
  out = mod(x, octree, depth)
  gout = torch.randn(out.shape, generator=g).to(dtype)
  out.backward(gout.to(DEV))
  want = layer(ref, f64(data), f64(mod.weights), depth, ks3, stride, nempty, bias=f64(mod.bias), grad=f64(gout))
  assert tuple(out.shape) == want[0].shape
  return {'out': rel_err(out, want[0]), 'gdata': rel_err(x.grad, want[1]), 'gw': rel_err(mod.weights.grad, want[2]),
          'gb': rel_err(mod.bias.grad, want[3])}


@pytest.mark.parametrize('kind', ['conv', 'deconv', 'dwconv'])
def test_layers_on_a_bare_octree(fixture, kind):
  d, ref = fixture
  bare = BareOctree(d, DEV)
  assert not isinstance(bare, Octree) and not hasattr(bare, '_table')
  seed = 0
  for ks, stride in (([3], 1), ([2], 2), ([3], 2), ([3, 1, 1], 1), ([3, 3, 1], 2)):
    for nempty in (False, True):
      for dtype, cin, cout in ((torch.float32, 5, 7), (torch.bfloat16, 32, 32), (torch.float16, 64, 64)):
        depth = 5 if kind == 'deconv' and stride == 2 else 6
        seed += 1
        say('bare octree', kind, ks, 'stride', stride, 'nempty', nempty, dtype, cin, cout, 'depth', depth)
        errs = run(kind, bare, ref, depth, ks, stride, nempty, cin, cout, dtype, seed)
        assert max(errs.values()) < TOL[dtype], (kind, ks, stride, nempty, dtype, errs)
  # one adapter per octree, kept with it, and none of the reference-side members was touched
  adapter = tables_of(bare)
  assert isinstance(adapter, ContractOctree) and tables_of(bare) is adapter and tables_of(adapter) is adapter
  assert bare.children[6].dtype == torch.int32 and bare.neighs[6].dtype == torch.int64


def test_bare_octree_with_int64_children_and_rebuilt_layers(fixture):
  """children of another integer type are converted; tables made from a layer's tensors are dropped
  when the octree replaces them (octree_grow, merge), and pad / depad take the bare octree too."""
  d, ref = fixture
  bare = BareOctree(d, DEV, child_dtype=torch.int64)
  errs = run('conv', bare, ref, 6, [2], 2, False, 32, 64, torch.bfloat16, 3)
  assert max(errs.values()) < TOL[torch.bfloat16], errs
  adapter = tables_of(bare)
  t0 = adapter._table(5, '333', 1, True)
  assert adapter._table(5, '333', 1, True) is t0
  want = bare.get_neigh(5, '333', 1, True)
  assert t0.dtype == torch.int32 and torch.equal(t0.long(), want)
  bare.neighs[5] = bare.neighs[5].clone()                    # "rebuilt": another tensor, same values
  t1 = adapter._table(5, '333', 1, True)
  assert t1 is not t0 and torch.equal(t1, t0)
  x = torch.randn(int(bare.nnum_nempty[5]), 8, device=DEV)
  padded = octree_pad(x, bare, 5)
  assert padded.shape[0] == int(bare.nnum[5]) and torch.equal(octree_depad(padded, bare, 5), x)
  np.testing.assert_array_equal(padded.cpu().numpy(), C.octree_pad(x.cpu().numpy(), ref, 5))


def test_bare_octree_on_the_cpu_is_refused(fixture):
  d, _ = fixture
  bare = BareOctree(d, 'cpu')
  conv = OctreeConv(4, 4, [3], 1).to(DEV)
  with pytest.raises(RuntimeError):
    conv(torch.randn(int(bare.nnum[6]), 4, device=DEV), bare, 6)
