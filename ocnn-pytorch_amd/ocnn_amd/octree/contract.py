"""Layers on an octree that only honours the public contract of the reference's class.

The modules need int32 tables, inverse tables, tile plans and the index of the non-empty
nodes.  `ocnn_amd.octree.Octree` keeps them itself.  Any other octree - the reference's own
class built on the CPU and moved to the GPU (ocnn/octree/octree.py:600-651,
ocnn/dataset.py:134-163), or an object that merely offers

    get_neigh(depth, kernel, stride, nempty) -> (rows, K) integer tensor, -1 = no neighbour
    children[depth]                          -> (nnum[depth],) int tensor, -1 = empty node
    nnum[depth], nnum_nempty[depth]

(ocnn/octree/octree.py:490-523 and :55-84; what ocnn/nn/octree_conv.py:51-100 reads) - gets a
`ContractOctree` beside it that derives the same things from those members and caches them
for as long as the octree keeps the tensors it was made from.
"""

import weakref

import torch

from .. import _lib
from .octree import LUT_INTERNAL, Octree, PlanHistory

_ADAPTERS = weakref.WeakKeyDictionary()
_ATTR = '_ocnn_amd_contract'


def tables_of(octree):
  """The object the layers ask for tables and plans: the octree itself when it is this
  package's, else the ContractOctree kept with it."""
  if isinstance(octree, (Octree, ContractOctree)):
    return octree
  adapter = getattr(octree, '__dict__', {}).get(_ATTR)
  if adapter is None:
    try:
      adapter = _ADAPTERS.get(octree)
    except TypeError:                     # not weakly referable
      adapter = None
  if adapter is None:
    adapter = ContractOctree(octree)
    try:
      octree.__dict__[_ATTR] = adapter
    except (AttributeError, TypeError):
      try:
        _ADAPTERS[octree] = adapter
      except TypeError:
        pass                              # nowhere to keep it: made again at the next call
  return adapter


class ContractOctree:
  """Tables, inverse tables, plans and non-empty index of a foreign octree, from its public
  members only.  Everything else (`nnum`, `keys`, ...) is the foreign octree's own."""

  # the plans asked for by earlier octrees of the same kind are built together on a fresh one
  plan_history = PlanHistory()

  def __init__(self, octree):
    self.__dict__['_o'] = octree
    self._tables, self._tables_t, self._plans = {}, {}, {}
    self._index32, self._children32, self._stamp = {}, {}, {}
    self._plans_prebuilt = False
    self.neighs = _Has(octree)

  def __getattr__(self, name):            # (only called for what the adapter does not hold)
    return getattr(self.__dict__['_o'], name)

  @property
  def depth(self):
    o = self._o
    return int(o.depth) if hasattr(o, 'depth') else len(o.children) - 1

  @property
  def full_depth(self):
    return int(getattr(self._o, 'full_depth', 2))

  # ---- validity: a layer of the foreign octree may be rebuilt (octree_grow, merge) ----------
  def _check(self, depth):
    """Forgets what was derived from tensors the octree no longer holds."""
    o = self._o
    child = o.children[depth]
    base = o.neighs[depth] if hasattr(o, 'neighs') else None
    stamp = tuple((id(t), t.data_ptr(), tuple(t.shape)) if t is not None else None for t in (child, base))
    if self._stamp.get(depth) != stamp:
      self._stamp[depth] = stamp
      for cache in (self._tables, self._tables_t):
        for key in [k for k in cache if k[0] == depth]:
          del cache[key]
      for key in [k for k in self._plans if k[0][0] == depth]:
        del self._plans[key]
      self._index32.pop(depth, None)
      self._children32.pop(depth, None)

  # ---- what the layers ask for -----------------------------------------------------------
  @property
  def children(self):
    return _Children(self)

  def _children_of(self, depth):
    self._check(depth)
    if depth not in self._children32:
      child = self._o.children[depth]
      _lib.require_gpu(child)
      self._children32[depth] = child.to(torch.int32).contiguous()
    return self._children32[depth]

  def _nempty_index32(self, depth):
    child = self._children_of(depth)
    if depth not in self._index32:
      n = int(self._o.nnum_nempty[depth])
      i32 = torch.empty(n, dtype=torch.int32, device=child.device)
      _lib.check(_lib.lib().ocnn_nempty_index(_lib.ptr(child), child.numel(), _lib.ptr(i32), None, _lib.stream()))
      self._index32[depth] = i32
    return self._index32[depth]

  def _table(self, depth, kernel='333', stride=1, nempty=False):
    """int32 copy of the octree's own get_neigh(depth, kernel, stride, nempty), cached."""
    self._check(depth)
    ck = (depth, kernel, stride, bool(nempty))
    if ck not in self._tables:
      if kernel in LUT_INTERNAL:          # (not a kernel of the contract: columns of its 3x3x3 table)
        cols = torch.tensor(LUT_INTERNAL[kernel], device=self._table(depth, '333', stride, nempty).device)
        self._tables[ck] = self._table(depth, '333', stride, nempty).index_select(1, cols).contiguous()
        return self._tables[ck]
      t = self._o.get_neigh(depth, kernel, stride, nempty)
      _lib.require_gpu(t)
      t = t.contiguous()
      if t.dtype == torch.int64:
        out = torch.empty(t.shape, dtype=torch.int32, device=t.device)
        _lib.check(_lib.lib().ocnn_table_to_i32(_lib.ptr(t), t.numel(), _lib.ptr(out), _lib.stream()))
        t = out
      else:
        t = t.to(torch.int32)
      self._tables[ck] = t
    return self._tables[ck]

  def _fine_rows(self, depth, nempty):
    return int(self._o.nnum_nempty[depth] if nempty else self._o.nnum[depth])

  # the inverse table and the plans are derived from _table exactly as for this package's octree
  _table_t = Octree._table_t
  _prebuild_plans = Octree._prebuild_plans

  def _plan(self, depth, kernel, stride, nempty, inverse=False, rows_in=None):
    self._check(depth)
    return Octree._plan(self, depth, kernel, stride, nempty, inverse, rows_in)


class _Children:
  """octree.children[d] as the int32 device tensor the kernels read."""

  def __init__(self, owner):
    self._owner = owner

  def __getitem__(self, depth):
    return self._owner._children_of(depth)

  def __len__(self):
    return len(self._owner._o.children)


class _Has:
  """`neighs.has(d)` of the foreign octree (what the prebuilding of plans asks)."""

  def __init__(self, octree):
    self._o = octree

  def has(self, depth):
    neighs = getattr(self._o, 'neighs', None)
    try:
      return neighs is None or neighs[depth] is not None
    except (IndexError, KeyError):
      return False
