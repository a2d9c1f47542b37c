"""Octree with the contract of the reference's ``ocnn.octree.Octree``
(ocnn/octree/octree.py), built and searched by HIP kernels.

Layout in device memory, per depth d:
  keys[d]      int64 (nnum[d],)      ascending Morton keys, batch id at bit 48
  children[d]  int32 (nnum[d],)      ordinal among the non-empty nodes, or -1
  neighs[d]    (nnum[d], 27)         row indices of the 3x3x3 window, or -1
The neighbour tables are kept as int32 (what the convolution kernels read);
``octree.neighs[d]`` widens one to the reference's int64 on first access.
nnum / nnum_nempty stay on the host, as in the reference.
"""

from typing import List, Union

import ctypes
import threading

import torch
import torch.nn.functional as F

from .. import _lib
from ..utils import cumsum, range_grid, trunc_div
from .points import Points
from .shuffled_key import key2xyz, xyz2key

LUT_KERNEL = {
    '222': [13, 14, 16, 17, 22, 23, 25, 26],
    '311': [4, 13, 22],
    '131': [10, 13, 16],
    '113': [12, 13, 14],
    '331': [1, 4, 7, 10, 13, 16, 19, 22, 25],
    '313': [3, 4, 5, 12, 13, 14, 21, 22, 23],
    '133': [9, 10, 11, 12, 13, 14, 15, 16, 17],
}
# tables the layers ask for on top of the reference's kernels: '222m', the mirror image of '222'
# (offsets {-1, 0}^3: where the fine neighbours of a first child live, seen from the coarse side)
LUT_INTERNAL = {
    '222m': [0, 1, 3, 4, 9, 10, 12, 13],
}


class _NeighTables:
  """List-like holder of the per-depth tables: int32 for the kernels, int64
  (the public dtype) made on demand and cached."""

  def __init__(self, num):
    self._t32 = [None] * num
    self._t64 = [None] * num

  def __len__(self):
    return len(self._t32)

  def _get(self, i):
    if self._t64[i] is None and self._t32[i] is not None:
      t32 = self._t32[i]
      if t32.is_cuda:
        out = torch.empty(t32.shape, dtype=torch.long, device=t32.device)
        _lib.check(_lib.lib().ocnn_table_to_i64(_lib.ptr(t32), t32.numel(), _lib.ptr(out),
                                                _lib.stream()))
      else:
        out = t32.long()
      self._t64[i] = out
    return self._t64[i]

  def __getitem__(self, i):
    if isinstance(i, slice):
      return [self._get(j) for j in range(*i.indices(len(self)))]
    return self._get(range(len(self))[i])

  def __setitem__(self, i, value):
    i = range(len(self))[i]
    self._t32[i] = self._t64[i] = None
    if value is None:
      return
    if value.dtype == torch.int32:
      self._t32[i] = value
    else:
      self._t64[i] = value.long()

  def __iter__(self):
    return (self._get(i) for i in range(len(self)))

  def append(self, value):
    self._t32.append(None)
    self._t64.append(None)
    self[len(self) - 1] = value

  def get32(self, i):
    if self._t32[i] is None and self._t64[i] is not None:
      t64 = self._t64[i].contiguous()
      if t64.is_cuda:
        out = torch.empty(t64.shape, dtype=torch.int32, device=t64.device)
        _lib.check(_lib.lib().ocnn_table_to_i32(_lib.ptr(t64), t64.numel(), _lib.ptr(out),
                                                _lib.stream()))
      else:
        out = t64.int()
      self._t32[i] = out
    return self._t32[i]

  def has(self, i):
    return self._t32[i] is not None or self._t64[i] is not None

  def moved(self, device, non_blocking=False):
    out = _NeighTables(len(self))
    for i in range(len(self)):
      if self._t32[i] is not None:
        out._t32[i] = self._t32[i].to(device, non_blocking=non_blocking)
      if self._t64[i] is not None:
        out._t64[i] = self._t64[i].to(device, non_blocking=non_blocking)
    return out


class TilePlan:
  """Per-tile distinct-row lists of a table (see ocnn_tile_plan_* in the C ABI).

  The kernels on the plan stage a tile's distinct rows in LDS and take tiles of up to `cap`
  rows.  A handful of denser tiles must not send a whole level to the plan-free kernels: when
  at most a tenth of the tiles are over the limit, those tiles are emptied in the plan (as if
  their table rows were all -1) and their rows listed in `overflow_rows` / `overflow_table`;
  the Python layer runs them through the plan-free kernels and puts the results in place.

  Building a plan needs sizes on the host (the length of the row lists); `build_many` makes
  the plans of several tables with ONE read-back for all of them, which is what a fresh octree
  in the middle of a training step wants: every read-back waits for the whole queue of kernels
  before it and leaves the device idle while the host catches up."""

  CAP = 415      # the smallest limit of the kernels on the plan
  LIST_PAD = 416  # rows a tile's list may have in the one-pass build

  def __init__(self, table: torch.Tensor, cap: int = None):
    self._count(table, cap)
    self._finish(self._host_stats(self._stats.tolist(), table, cap))

  def _host_stats(self, stats, table, cap):
    """The sizes on the host; a table the one-pass build gave up on (tiles with more distinct
    blocks of rows than its set holds: no locality) is counted again the long way first."""
    if stats[5]:
      self._count(table, cap, one_pass=False)
      stats = self._stats.tolist()
    return [int(v) for v in stats]

  @classmethod
  def build_many(cls, tables, cap: int = None):
    """Plans of several tables with one device -> host read-back."""
    plans = [cls.__new__(cls) for _ in tables]
    for p, t in zip(plans, tables):
      p._count(t, cap)
    host = torch.stack([p._stats for p in plans]).tolist() if plans else []
    for p, t, st in zip(plans, tables, host):
      p._finish(p._host_stats(st, t, cap))
    return plans

  def _count(self, table, cap, one_pass=True):
    """First half: distinct rows per tile, their offsets, and the sizes the second half
    needs on the host as one device vector."""
    _lib.require_gpu(table)
    L = _lib.lib()
    table = table.contiguous()
    rows, K = table.shape
    self._tile_rows = L.ocnn_tile_plan_rows()
    tiles = (rows + self._tile_rows - 1) // self._tile_rows
    self._cap = self.CAP if cap is None else cap
    self._table = table
    self.rows, self.K = rows, K
    self.overflow_rows = self.overflow_table = None
    self._pairs = None
    self._on_pairs = None          # called when the pair plan is first asked for
    dev, st = table.device, _lib.stream()
    self._ucount = torch.empty(tiles, dtype=torch.int32, device=dev)
    tile_nnz = torch.empty(tiles, dtype=torch.int32, device=dev)
    self.uptr = torch.empty(tiles + 1, dtype=torch.int32, device=dev)
    self._stats = torch.empty(6, dtype=torch.int64, device=dev)
    # One pass over the table: counts, positions and the lists at fixed places (LIST_PAD rows a
    # tile); the second half only moves the lists to their offsets.  (A limit above LIST_PAD, or
    # a table whose tiles do not fit it, takes the two passes of count and fill.)
    self._lists = None
    if one_pass and self._cap <= self.LIST_PAD:
      self._lists = torch.empty(max(tiles, 1) * self.LIST_PAD, dtype=torch.int32, device=dev)
      # uint16 payload, [tile][slot][row in tile]: whole tiles, the tail reads "empty"
      self.loc = torch.empty((tiles, K, self._tile_rows), dtype=torch.int16, device=dev)
      _lib.check(L.ocnn_tile_plan_build(_lib.ptr(table), rows, K, self.LIST_PAD, _lib.ptr(self._ucount),
                                        _lib.ptr(tile_nnz), _lib.ptr(self._lists), _lib.ptr(self.loc), st))
    else:
      _lib.check(L.ocnn_tile_plan_count(_lib.ptr(table), rows, K, _lib.ptr(self._ucount), _lib.ptr(tile_nnz), st))
    _lib.check(L.ocnn_tile_plan_offsets(_lib.ptr(self._ucount), _lib.ptr(tile_nnz), tiles, self._cap,
                                        _lib.ptr(self.uptr), _lib.ptr(self._stats), st))

  def _finish(self, stats):
    """Second half, with the sizes on the host: row lists and positions."""
    L = _lib.lib()
    table, tile_rows = self._table, self._tile_rows
    rows, K = self.rows, self.K
    tiles = self._ucount.numel()
    dev = table.device
    _, dropped, total, umax, nnz = stats[:5]
    one_pass = self._lists is not None and umax <= self.LIST_PAD
    if dropped:
      big = self._ucount > self._cap
      idx = (big.nonzero().view(-1, 1) * tile_rows + torch.arange(tile_rows, device=dev).view(1, -1)).view(-1)
      idx = idx[idx < rows]
      self.overflow_rows = idx
      self.overflow_table = table.index_select(0, idx).contiguous()
      if not one_pass:
        table = table.clone()
        table[idx] = -1
    # how often a staged row is used by its tile: near 1 there is nothing to gain from staging
    self.reuse = nnz / max(total, 1)
    self.urows = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
    if one_pass:
      _lib.check(L.ocnn_tile_plan_compact(_lib.ptr(self._ucount), _lib.ptr(self.uptr), _lib.ptr(self._stats),
                                          self._cap, self.LIST_PAD, _lib.ptr(self._lists), _lib.ptr(self.urows),
                                          _lib.ptr(self.loc), K, tiles, _lib.stream()))
    else:
      # uint16 payload, [tile][slot][row in tile]: whole tiles, the tail reads "empty"
      self.loc = torch.empty((tiles, K, tile_rows), dtype=torch.int16, device=dev)
      _lib.check(L.ocnn_tile_plan_fill(_lib.ptr(table), rows, K, _lib.ptr(self.uptr),
                                       _lib.ptr(self.urows), _lib.ptr(self.loc), _lib.stream()))
    self.total, self.umax, self.nnz = total, umax, nnz
    self._table = self._ucount = self._stats = self._lists = None

  @property
  def occupancy(self):
    """Share of the table's entries that hold a row."""
    return self.nnz / max(self.rows * self.K, 1)

  def pairs(self):
    """Pair plan of the table for ocnn_conv_gather_sparse (built on first use): per tile
    and slot the rows that have a neighbour, in blocks of 16 entries."""
    if self._pairs is None:
      self._pairs = PairPlan(self)
      if self._on_pairs is not None:
        self._on_pairs()
    return self._pairs


class PairPlan:
  """Blocks of 16 (row, neighbour) pairs per tile and list of a table; a list is a slot, or
  a range of the tiles' rows of a slot with many pairs; the lists are dealt to four groups
  of about equal numbers of pairs (see ocnn_pair_plan_* in the C ABI).  `build_many` makes
  the pair plans of several tile plans with two read-backs in all."""

  def __init__(self, plan: TilePlan):
    self._slot_counts(plan)
    self._lists(self._counts.tolist())
    self._finish([int(v) for v in self._sizes.tolist()] if self._sizes is not None else None)

  @classmethod
  def build_many(cls, plans):
    out = [cls.__new__(cls) for _ in plans]
    for pp, plan in zip(out, plans):
      pp._slot_counts(plan)
    host = torch.cat([pp._counts for pp in out]).tolist() if out else []
    at = 0
    for pp in out:
      pp._lists(host[at:at + pp._K])
      at += pp._K
    sizes = [pp._sizes for pp in out if pp._sizes is not None]
    host = torch.stack(sizes).tolist() if sizes else []
    it = iter(host)
    for pp in out:
      pp._finish([int(v) for v in next(it)] if pp._sizes is not None else None)
    return out

  def _slot_counts(self, plan):
    L = _lib.lib()
    self._plan = plan
    self._tiles, self._K, _ = plan.loc.shape
    self._counts = torch.zeros(self._K, dtype=torch.int64, device=plan.loc.device)
    _lib.check(L.ocnn_pair_plan_slot_counts(_lib.ptr(plan.loc), self._tiles, self._K, _lib.ptr(self._counts),
                                            _lib.stream()))

  def _lists(self, counts):
    """With the pairs per slot on the host: the lists and their groups, then the number of
    blocks per (tile, list)."""
    L = _lib.lib()
    plan, tiles, K = self._plan, self._tiles, self._K
    dev = plan.loc.device
    per_slot = (ctypes.c_int64 * K)(*[int(c) for c in counts])
    # host arrays, kept alive with the plan: the C ABI reads them at every call
    self.lists_host = (ctypes.c_int32 * 32)()
    self.list_count_host = (ctypes.c_int64 * 32)()
    self.group_bounds_host = (ctypes.c_int32 * 5)()
    n_lists = ctypes.c_int(0)
    _lib.check(L.ocnn_pair_plan_lists(K, ctypes.addressof(per_slot), ctypes.addressof(self.lists_host),
                                      ctypes.addressof(self.list_count_host),
                                      ctypes.addressof(self.group_bounds_host), ctypes.addressof(n_lists)))
    nl = self.n_lists = n_lists.value
    self.lists = torch.tensor(list(self.lists_host)[:nl], dtype=torch.int32).to(dev, non_blocking=True)
    nblk = torch.zeros(max(tiles * nl, 1), dtype=torch.int32, device=dev)
    _lib.check(L.ocnn_pair_plan_count(_lib.ptr(plan.loc), tiles, K, _lib.ptr(self.lists), nl, _lib.ptr(nblk),
                                      _lib.stream()))
    self.cptr = torch.zeros(tiles * nl + 1, dtype=torch.int32, device=dev)
    self._sizes = None
    if tiles > 0:
      self.cptr[1:] = torch.cumsum(nblk[:tiles * nl], 0)
      self._sizes = torch.stack([self.cptr[-1], nblk[:tiles * nl].view(tiles, nl).sum(1).max().int()])

  def _finish(self, sizes):
    L = _lib.lib()
    plan = self._plan
    self.n_blocks, self.max_blocks = sizes if sizes is not None else (0, 0)
    self.ent = torch.empty(max(self.n_blocks, 1) * 16, dtype=torch.int32, device=plan.loc.device)
    _lib.check(L.ocnn_pair_plan_fill(_lib.ptr(plan.loc), self._tiles, self._K, _lib.ptr(self.lists), self.n_lists,
                                     _lib.ptr(self.cptr), _lib.ptr(self.ent), _lib.stream()))
    self._plan = self._counts = self._sizes = None


class PlanHistory:
  """Which tile plans (and pair plans) octrees of a kind (depth, full_depth) were asked for.
  Bounded (the kinds and the plans of a kind seen least recently are dropped) and safe to
  use from several threads."""

  MAX_KINDS = 16
  MAX_PLANS = 64

  def __init__(self):
    self._lock = threading.Lock()
    self._kinds = {}           # kind -> {plan key: pair plan wanted}, both in order of last use

  def requests(self, kind):
    """Snapshot {plan key: pair plan wanted} of a kind."""
    with self._lock:
      return dict(self._kinds.get(kind, {}))

  def note(self, kind, key, pairs=False):
    with self._lock:
      plans = self._kinds.pop(kind, {})
      plans[key] = plans.pop(key, False) or pairs
      while len(plans) > self.MAX_PLANS:
        plans.pop(next(iter(plans)))
      self._kinds[kind] = plans
      while len(self._kinds) > self.MAX_KINDS:
        self._kinds.pop(next(iter(self._kinds)))

  def clear(self):
    with self._lock:
      self._kinds.clear()


class Octree:
  """Same constructor, attributes and methods as the reference class
  (ocnn/octree/octree.py:18-106)."""

  def __init__(self, depth: int, full_depth: int = 2, batch_size: int = 1,
               device: Union[torch.device, str] = 'cpu', **kwargs):
    self.depth = depth
    self.full_depth = full_depth
    self.batch_size = batch_size
    self.device = device
    self.reset()

  def reset(self):
    num = self.depth + 1
    self.keys = [None] * num
    self.children = [None] * num
    self.neighs = _NeighTables(num)
    self.features = [None] * num
    self.normals = [None] * num
    self.points = [None] * num
    self.nempty_masks = [None] * num
    self.nempty_indices = [None] * num
    self.nempty_neighs = [None] * num
    self._nempty_indices32 = [None] * num
    self._tables = {}        # (depth, kernel, stride, nempty) -> int32 table
    self._tables_t = {}      # same key -> inverse table
    self._plans = {}         # (key, inverse) -> TilePlan
    self._plans_prebuilt = False

    self.nnum = torch.zeros(num, dtype=torch.long)
    self.nnum_nempty = torch.zeros(num, dtype=torch.long)
    bs = self.batch_size
    self.batch_nnum = torch.zeros(num, bs, dtype=torch.long)
    self.batch_nnum_nempty = torch.zeros(num, bs, dtype=torch.long)

    # the reference's public lookup tables (ocnn/octree/octree.py:85-106); the
    # kernels compute the first two arithmetically
    dev = self.device
    grid = range_grid(2, 3, dev).unsqueeze(1) + range_grid(-1, 1, dev)
    self.lut_parent = (trunc_div(grid, 2) * torch.tensor([9, 3, 1], device=dev)).sum(2)
    self.lut_child = ((grid % 2) * torch.tensor([4, 2, 1], device=dev)).sum(2)
    self.lut_kernel = {k: torch.tensor(v, device=dev) for k, v in LUT_KERNEL.items()}

  # ---- cache bookkeeping ---------------------------------------------------
  def _drop_tables(self, depth, nempty_only=False):
    for cache in (self._tables, self._tables_t):
      for key in [k for k in cache if k[0] == depth and (k[3] or not nempty_only)]:
        del cache[key]
    for key in [k for k in self._plans if k[0][0] == depth and (k[0][3] or not nempty_only)]:
      del self._plans[key]

  def _drop_nempty(self, depth):
    self.nempty_masks[depth] = None
    self.nempty_indices[depth] = None
    self.nempty_neighs[depth] = None
    self._nempty_indices32[depth] = None
    self._drop_tables(depth, nempty_only=True)

  # ---- simple accessors (ocnn/octree/octree.py:108-145) ---------------------
  def key(self, depth: int, nempty: bool = False):
    key = self.keys[depth]
    return key[self.nempty_index(depth)] if nempty else key

  def xyzb(self, depth: int, nempty: bool = False):
    return key2xyz(self.key(depth, nempty), depth)

  def batch_id(self, depth: int, nempty: bool = False):
    batch_id = self.keys[depth] >> 48
    return batch_id[self.nempty_index(depth)] if nempty else batch_id

  # ---- non-empty bookkeeping (ocnn/octree/octree.py:147-199) ----------------
  def nempty_mask(self, depth: int, reset: bool = False):
    if self.nempty_masks[depth] is None or reset:
      self.nempty_masks[depth] = self.children[depth] >= 0
    return self.nempty_masks[depth]

  def _make_nempty_index(self, depth):
    child = self.children[depth]
    _lib.require_gpu(child)
    n = int(self.nnum_nempty[depth])
    i32 = torch.empty(n, dtype=torch.int32, device=child.device)
    i64 = torch.empty(n, dtype=torch.long, device=child.device)
    _lib.check(_lib.lib().ocnn_nempty_index(_lib.ptr(child), child.numel(), _lib.ptr(i32),
                                            _lib.ptr(i64), _lib.stream()))
    self._nempty_indices32[depth] = i32
    self.nempty_indices[depth] = i64

  def nempty_index(self, depth: int, reset: bool = False):
    if self.nempty_indices[depth] is None or reset:
      if not reset and self._nempty_indices32[depth] is not None:
        self.nempty_indices[depth] = self._nempty_indices32[depth].long()
      else:
        self._make_nempty_index(depth)
    return self.nempty_indices[depth]

  def _nempty_index32(self, depth):
    if self._nempty_indices32[depth] is None:
      self._make_nempty_index(depth)
    return self._nempty_indices32[depth]

  def nempty_neigh(self, depth: int, reset: bool = False):
    if self.nempty_neighs[depth] is None or reset:
      if reset:
        self._drop_tables(depth, nempty_only=True)
      self.nempty_neighs[depth] = self._widen(self._table(depth, '333', 1, True))
    return self.nempty_neighs[depth]

  def remap_nempty_neigh(self, neigh: torch.Tensor, depth: int):
    """In-place remap of valid entries to non-empty ordinals
    (ocnn/octree/octree.py:188-199)."""
    valid = neigh >= 0
    neigh[valid] = self.children[depth][neigh[valid]].long()
    return neigh

  # ---- build (ocnn/octree/octree.py:201-287) --------------------------------
  def build_octree(self, point_cloud: Points, bbmin: Union[float, torch.Tensor] = -1.0,
                   bbmax: Union[float, torch.Tensor] = 1.0):
    self.device = point_cloud.device
    assert point_cloud.batch_size == self.batch_size, 'Inconsistent batch_size'
    pts = point_cloud.points
    _lib.require_gpu(pts)
    L = _lib.lib()
    dev = pts.device
    depth = self.depth

    # normalisation constants exactly as Points.normalize forms them
    box = bbmax - bbmin
    if type(box) is torch.Tensor:
      box = box.max().item()
    assert box > 0, 'The bounding box size must be greater than 0.'
    factor = (2 ** depth) / box
    if isinstance(bbmin, torch.Tensor):
      lo = [float(v) for v in bbmin.detach().float().cpu().view(-1).tolist()]
      lo = lo * 3 if len(lo) == 1 else lo
    else:
      lo = [float(bbmin)] * 3
    h_lo = (ctypes.c_float * 3)(*lo)

    pts = pts.float().contiguous()
    npt = pts.shape[0]
    batch, batch_is_float = None, 0
    if self.batch_size > 1:
      batch = point_cloud.batch_id.view(-1)
      if batch.is_floating_point():
        batch, batch_is_float = batch.float().contiguous(), 1
      else:
        batch = batch.long().contiguous()
    pts_norm = torch.empty_like(pts)
    key = torch.empty(npt, dtype=torch.long, device=dev)
    st = _lib.stream()
    _lib.check(L.ocnn_points2key(_lib.ptr(pts), npt, h_lo, factor, _lib.ptr(batch),
                                 batch_is_float, depth, _lib.ptr(pts_norm), _lib.ptr(key), st))

    # sort, then every layer's node numbering in one scan: one read-back for the whole build
    full_depth = self.full_depth
    levels = depth - full_depth
    batch_bits = max(0, (self.batch_size - 1).bit_length())
    ws = _lib.workspace(L.ocnn_octree_build_workspace_bytes(npt, depth, full_depth, batch_bits), dev)
    perm = torch.empty(npt, dtype=torch.int32, device=dev)
    sizes = torch.empty(levels + 1, dtype=torch.long, device=dev)
    _lib.check(L.ocnn_octree_build_scan(_lib.ptr(key), npt, depth, full_depth, batch_bits,
                                        _lib.ptr(ws), ws.numel(), _lib.ptr(perm), _lib.ptr(sizes),
                                        st))
    # what does not wait for the sizes is allocated while the sort runs
    full = [self.batch_size << (3 * d) for d in range(full_depth + 1)]
    for d in range(full_depth + 1):
      self.keys[d] = torch.empty(full[d], dtype=torch.long, device=dev)
      self.children[d] = torch.empty(full[d], dtype=torch.int32, device=dev)
    idx = torch.empty(npt, dtype=torch.long, device=dev)
    seg_start = torch.empty(npt + 1, dtype=torch.int32, device=dev)
    sizes = sizes.tolist()
    nleaf = sizes[0]

    nnum = full + [8 * sizes[depth - d + 1] for d in range(full_depth + 1, depth + 1)]
    for d in range(full_depth + 1, depth + 1):
      self.keys[d] = torch.empty(nnum[d], dtype=torch.long, device=dev)
      self.children[d] = torch.empty(nnum[d], dtype=torch.int32, device=dev)
    h_sizes = (ctypes.c_int64 * (levels + 1))(*sizes)
    h_keys = (ctypes.c_void_p * (depth + 1))(*[t.data_ptr() for t in self.keys[:depth + 1]])
    h_children = (ctypes.c_void_p * (depth + 1))(*[t.data_ptr() for t in self.children[:depth + 1]])
    _lib.check(L.ocnn_octree_build_fill(_lib.ptr(ws), npt, depth, full_depth, self.batch_size,
                                        batch_bits, h_sizes, _lib.ptr(perm), h_keys, h_children,
                                        _lib.ptr(idx), _lib.ptr(seg_start), st))

    # per-leaf signals
    def leaf(src, mode):
      src = src.float().contiguous()
      out = torch.empty(nleaf, src.shape[1], dtype=torch.float32, device=dev)
      _lib.check(L.ocnn_leaf_average(_lib.ptr(src), src.shape[1], _lib.ptr(perm),
                                     _lib.ptr(seg_start), nleaf, mode, _lib.ptr(out), st))
      return out

    self.nnum[:depth + 1] = torch.tensor(nnum, dtype=torch.long)
    self.nnum_nempty[:depth + 1] = torch.tensor(
        full[:-1] + [sizes[depth - d] for d in range(full_depth, depth + 1)], dtype=torch.long)
    if point_cloud.normals is not None:
      nrm = point_cloud.normals.float().contiguous()
      self.points[depth] = torch.empty(nleaf, 3, dtype=torch.float32, device=dev)
      self.normals[depth] = torch.empty(nleaf, 3, dtype=torch.float32, device=dev)
      _lib.check(L.ocnn_leaf_points_normals(_lib.ptr(pts_norm), _lib.ptr(nrm), _lib.ptr(perm), _lib.ptr(seg_start),
                                            nleaf, _lib.ptr(self.points[depth]), _lib.ptr(self.normals[depth]), st))
    else:
      self.points[depth] = leaf(pts_norm, 0)
    if point_cloud.features is not None:
      self.features[depth] = leaf(point_cloud.features, 0)

    num = depth + 1
    self.nempty_masks = [None] * num
    self.nempty_indices = [None] * num
    self.nempty_neighs = [None] * num
    self._nempty_indices32 = [None] * num
    self._tables, self._tables_t, self._plans = {}, {}, {}
    self._plans_prebuilt = False
    return idx

  def _grow_full(self, depth: int, with_children: bool = True):
    num = self.batch_size << (3 * depth)
    self.nnum[depth] = num
    self.nnum_nempty[depth] = num
    dev = torch.device(self.device)
    if dev.type != 'cuda':
      raise RuntimeError('ocnn_amd builds octrees on the GPU only (device=%s)' % (dev,))
    keys = torch.empty(num, dtype=torch.long, device=dev)
    children = torch.empty(num, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
      _lib.check(_lib.lib().ocnn_build_full_layer(depth, self.batch_size, int(with_children),
                                                  _lib.ptr(keys), _lib.ptr(children),
                                                  _lib.stream()))
    self.keys[depth] = keys
    self.children[depth] = children

  def octree_grow_full(self, depth: int, update_neigh: bool = True):
    """Dense layer (ocnn/octree/octree.py:289-321)."""
    assert depth <= self.full_depth, 'error'
    self._grow_full(depth)
    self._drop_nempty(depth)
    if update_neigh:
      self.construct_neigh(depth)

  def octree_split(self, split: torch.Tensor, depth: int):
    """Declares which nodes of `depth` have children: `split` holds one number per node, non
    zero = split (ocnn/octree/octree.py:323-351).  One scan kernel numbers the split nodes;
    the count comes back with one read."""
    n = int(split.shape[0])
    assert n == int(self.nnum[depth]), 'one split decision per node of the layer'
    L = _lib.lib()
    flags = (split != 0).to(torch.int32).contiguous()
    _lib.require_gpu(flags)
    children = torch.empty(n, dtype=torch.int32, device=flags.device)
    count = torch.zeros(1, dtype=torch.long, device=flags.device)
    ws = _lib.workspace(L.ocnn_build_level_workspace_bytes(n), flags.device)
    _lib.check(L.ocnn_split_children(_lib.ptr(flags), n, _lib.ptr(ws), ws.numel(), _lib.ptr(children),
                                     _lib.ptr(count), _lib.stream()))
    self.children[depth] = children
    self.nnum_nempty[depth] = int(count)
    self._drop_nempty(depth)

  def _append_layer(self):
    """Room for one more layer in every per-depth list and count."""
    self.depth += 1
    for per_depth in (self.keys, self.children, self.features, self.normals, self.points, self.nempty_masks,
                      self.nempty_indices, self.nempty_neighs, self._nempty_indices32, self.neighs):
      per_depth.append(None)
    self.nnum = torch.cat([self.nnum, self.nnum.new_zeros(1)])
    self.nnum_nempty = torch.cat([self.nnum_nempty, self.nnum_nempty.new_zeros(1)])
    self.batch_nnum = torch.cat([self.batch_nnum, self.batch_nnum.new_zeros(1, self.batch_size)])
    self.batch_nnum_nempty = torch.cat([self.batch_nnum_nempty, self.batch_nnum_nempty.new_zeros(1, self.batch_size)])

  def octree_grow(self, depth: int, update_neigh: bool = True):
    """Creates layer `depth` as the children of the non-empty nodes of the layer above it, all
    of them marked non-empty until octree_split says otherwise
    (ocnn/octree/octree.py:353-402); the octree gets one layer deeper when needed."""
    if depth > self.depth:
      assert depth == self.depth + 1, 'layers are grown one at a time'
      self._append_layer()
    parents = int(self.nnum_nempty[depth - 1])
    total = 8 * parents
    above = self.keys[depth - 1]
    _lib.require_gpu(above)
    keys = torch.empty(total, dtype=torch.long, device=above.device)
    children = torch.empty(total, dtype=torch.int32, device=above.device)
    _lib.check(_lib.lib().ocnn_grow_layer(_lib.ptr(above), _lib.ptr(self._nempty_index32(depth - 1)), parents,
                                          _lib.ptr(keys), _lib.ptr(children), _lib.stream()))
    self.keys[depth], self.children[depth] = keys, children
    self.nnum[depth] = self.nnum_nempty[depth] = total
    self._drop_nempty(depth)
    if update_neigh:
      self.construct_neigh(depth)

  # ---- neighbour search (ocnn/octree/octree.py:404-446) ---------------------
  def construct_neigh(self, depth: int):
    L = _lib.lib()
    dev = torch.device(self.device) if isinstance(self.device, str) else self.device
    if dev.type != 'cuda':
      raise RuntimeError('ocnn_amd kernels need the octree on a HIP device, it is on '
                         '{}'.format(dev))
    st = _lib.stream()
    if depth <= self.full_depth:
      rows = self.batch_size << (3 * depth)
      out = torch.empty(rows, 27, dtype=torch.int32, device=dev)
      _lib.check(L.ocnn_neigh_full(depth, self.batch_size, None, _lib.ptr(out), st))
    else:
      child_p = self.children[depth - 1]
      neigh_p = self.neighs.get32(depth - 1)
      assert neigh_p is not None, 'construct_neigh({}) first'.format(depth - 1)
      n_ne = int(self.nnum_nempty[depth - 1])
      assert 8 * n_ne == int(self.nnum[depth]), 'octree layers are inconsistent'
      out = torch.empty(8 * n_ne, 27, dtype=torch.int32, device=dev)
      _lib.check(L.ocnn_neigh_from_parent(_lib.ptr(child_p), _lib.ptr(neigh_p.contiguous()),
                                          _lib.ptr(self._nempty_index32(depth - 1)), n_ne, None,
                                          _lib.ptr(out), st))
    self.neighs[depth] = out
    self.nempty_neighs[depth] = None
    self._drop_tables(depth)

  def construct_all_neigh(self):
    """All tables with one library call (ocnn/octree/octree.py:443-446): the launches of the
    shallow layers follow each other without the host in between."""
    dev = torch.device(self.device) if isinstance(self.device, str) else self.device
    depth = self.depth
    nnum = [int(v) for v in self.nnum[:depth + 1].tolist()]
    nempty = [int(v) for v in self.nnum_nempty[:depth + 1].tolist()]
    if dev.type != 'cuda' or self.full_depth < 1 or any(c is None for c in self.children[:depth + 1]) or \
        min(nnum[1:] + nempty) <= 0 or \
        any(nnum[d] != (self.batch_size << (3 * d) if d <= self.full_depth else 8 * nempty[d - 1])
            for d in range(1, depth + 1)):
      for d in range(1, depth + 1):                       # the layer-by-layer route says what is wrong
        self.construct_neigh(d)
      return
    neigh = [None] + [torch.empty(nnum[d], 27, dtype=torch.int32, device=dev) for d in range(1, depth + 1)]
    index = [torch.empty(nempty[d], dtype=torch.int32, device=dev) if self.full_depth <= d < depth else None
             for d in range(depth + 1)]
    ptrs = lambda ts: (ctypes.c_void_p * (depth + 1))(*[None if t is None else t.data_ptr() for t in ts])
    with torch.cuda.device(dev):
      _lib.check(_lib.lib().ocnn_neigh_all(depth, self.full_depth, self.batch_size,
                                           (ctypes.c_int64 * (depth + 1))(*nnum),
                                           (ctypes.c_int64 * (depth + 1))(*nempty), ptrs(self.children[:depth + 1]),
                                           ptrs(index), ptrs(neigh), _lib.stream()))
    for d in range(1, depth + 1):
      self.neighs[d] = neigh[d]
      self.nempty_neighs[d] = None
      self._drop_tables(d)
    for d in range(self.full_depth, depth):
      self._nempty_indices32[d] = index[d]
      self.nempty_indices[d] = None

  # ---- search (ocnn/octree/octree.py:448-488) -------------------------------
  def search_xyzb(self, query: torch.Tensor, depth: int, nempty: bool = False):
    key = xyz2key(query[:, 0], query[:, 1], query[:, 2], query[:, 3], depth)
    return self.search_key(key, depth, nempty)

  def search_key(self, query: torch.Tensor, depth: int, nempty: bool = False):
    key = self.key(depth, nempty).contiguous()
    _lib.require_gpu(key, query)
    query = query.to(torch.long).contiguous()
    idx = torch.empty(query.shape, dtype=torch.long, device=query.device)
    _lib.check(_lib.lib().ocnn_search_key(_lib.ptr(key), key.numel(), _lib.ptr(query), query.numel(),
                                          _lib.ptr(idx), _lib.stream()))
    return idx

  # ---- tables for the layers ------------------------------------------------
  def _table(self, depth, kernel='333', stride=1, nempty=False):
    """int32 table of get_neigh(depth, kernel, stride, nempty), cached."""
    if stride not in (1, 2):
      raise ValueError('Unsupported stride {}'.format(stride))
    if kernel != '333' and kernel not in LUT_KERNEL and kernel not in LUT_INTERNAL:
      raise ValueError('Unsupported kernel {}'.format(kernel))
    ck = (depth, kernel, stride, bool(nempty))
    if ck in self._tables:
      return self._tables[ck]
    base = self.neighs.get32(depth)
    assert base is not None, 'construct_neigh({}) first'.format(depth)
    if kernel == '333' and stride == 1 and not nempty:
      self._tables[ck] = base
      return base
    _lib.require_gpu(base)
    if kernel == '222' and stride == 2 and nempty and self.children[depth].numel() == base.shape[0]:
      # the 2x2x2 window of a parent's first child is its eight children, and the non-empty
      # numbering of node 8 p + c is children[8 p + c]: the table is a view of that array
      self._tables[ck] = self.children[depth].view(-1, 8)
      return self._tables[ck]
    cols = LUT_KERNEL.get(kernel, LUT_INTERNAL.get(kernel))
    K = 27 if cols is None else len(cols)
    h_cols = None if cols is None else (ctypes.c_int * K)(*cols)
    row_index, row_stride, rows = None, 1, base.shape[0]
    if stride == 2:
      row_stride, rows = 8, base.shape[0] // 8
    elif nempty:
      row_index, rows = self._nempty_index32(depth), int(self.nnum_nempty[depth])
    children = self.children[depth] if nempty else None
    out = torch.empty(rows, K, dtype=torch.int32, device=base.device)
    _lib.check(_lib.lib().ocnn_neigh_select(
        _lib.ptr(base), _lib.ptr(row_index), row_stride, _lib.ptr(children), h_cols, K, rows,
        None, _lib.ptr(out), _lib.stream()))
    self._tables[ck] = out
    return out

  def _table_t(self, depth, kernel, stride, nempty, rows_in):
    """Inverse table: row j, slot k -> the row i with table[i][k] == j."""
    ck = (depth, kernel, stride, bool(nempty))
    if ck not in self._tables_t:
      t = self._table(depth, kernel, stride, nempty)
      out = torch.empty(rows_in, t.shape[1], dtype=torch.int32, device=t.device)
      _lib.check(_lib.lib().ocnn_table_transpose(_lib.ptr(t), t.shape[0], t.shape[1], rows_in,
                                                 _lib.ptr(out), _lib.stream()))
      self._tables_t[ck] = out
    return self._tables_t[ck]

  # Plans asked for by earlier octrees of the same (depth, full_depth): a network asks every
  # octree for the same plans, layer by layer, and each plan built on its own costs two
  # device -> host read-backs in the middle of the step.  The first request on a fresh octree
  # therefore builds all the plans that `plan_history` holds for its kind, together.  The
  # history is an object: the default one is shared by all octrees of the process; an octree
  # (or a data loader, for all the octrees of one network) may carry its own
  # (`octree.plan_history = PlanHistory()`), and `clear()` forgets what was asked for.
  PREBUILD_PLANS = True
  plan_history = None        # set below to the process-wide default PlanHistory()

  def _plan(self, depth, kernel, stride, nempty, inverse=False, rows_in=None):
    """Tile plan of the table (or of its inverse), cached with the table."""
    ck = ((depth, kernel, stride, bool(nempty)), bool(inverse))
    if ck not in self._plans:
      history, kind = self.plan_history, (self.depth, self.full_depth)
      requests = history.requests(kind)
      if Octree.PREBUILD_PLANS and requests and not self._plans_prebuilt:
        self._plans_prebuilt = True
        self._prebuild_plans(requests)
      if ck not in self._plans:
        t = (self._table_t(depth, kernel, stride, nempty, rows_in) if inverse
             else self._table(depth, kernel, stride, nempty))
        self._plans[ck] = TilePlan(t)
      if rows_in is None or rows_in == self._fine_rows(depth, nempty):
        history.note(kind, ck)
        plan = self._plans[ck]
        if plan._pairs is None:
          plan._on_pairs = lambda: history.note(kind, ck, pairs=True)
    return self._plans[ck]

  def prepare(self):
    """Builds now, together, the tables and plans that earlier octrees of the same (depth,
    full_depth) were asked for (`plan_history`): what the first layer's request would otherwise
    set off in the middle of a step.  A training loop calls it on a side stream while the step
    before is still running,

      with torch.cuda.stream(side):
        nxt = Octree(...); nxt.build_octree(points); nxt.construct_all_neigh(); nxt.prepare()
      ...
      torch.cuda.current_stream().wait_stream(side)
      nxt.record_stream(torch.cuda.current_stream())

    so that a new octree every step costs the step nothing but the compute units its kernels
    take.  (No counterpart in the reference, whose data loader builds octrees on the CPU in
    worker processes: ocnn/dataset.py:61-67.)"""
    requests = self.plan_history.requests((self.depth, self.full_depth))
    if Octree.PREBUILD_PLANS and requests and not self._plans_prebuilt:
      self._plans_prebuilt = True
      self._prebuild_plans(requests)
    return self

  def record_stream(self, stream):
    """Tells torch's allocator that `stream` uses every device tensor this octree holds now
    (keys, children, tables, plans, leaf signals): for an octree built on another stream, so
    that its memory is not handed out again on that stream while work queued on `stream`
    still reads it."""
    seen = set()

    def walk(v):
      if id(v) in seen:
        return
      seen.add(id(v))
      if isinstance(v, torch.Tensor):
        if v.is_cuda:
          v.record_stream(stream)
      elif isinstance(v, (list, tuple)):
        for x in v:
          walk(x)
      elif isinstance(v, dict):
        for x in v.values():
          walk(x)
      elif isinstance(v, (TilePlan, PairPlan, _NeighTables)):
        walk(vars(v))

    walk(vars(self))
    return self

  def _fine_rows(self, depth, nempty):
    """Rows on the side of a table that its entries index (all tables of this class: the
    nodes of `depth`, or the non-empty ones)."""
    return int(self.nnum_nempty[depth] if nempty else self.nnum[depth])

  def _prebuild_plans(self, requests):
    keys = [ck for ck in requests if ck not in self._plans and ck[0][0] <= self.depth and
            self.neighs.has(ck[0][0])]
    tables = []
    for (depth, kernel, stride, nempty), inverse in keys:
      tables.append(self._table_t(depth, kernel, stride, nempty, self._fine_rows(depth, nempty)) if inverse
                    else self._table(depth, kernel, stride, nempty))
    plans = TilePlan.build_many(tables)
    for ck, plan in zip(keys, plans):
      self._plans[ck] = plan
    with_pairs = [plan for ck, plan in zip(keys, plans) if requests[ck]]
    for plan, pp in zip(with_pairs, PairPlan.build_many(with_pairs)):
      plan._pairs = pp

  @staticmethod
  def _widen(t32):
    out = torch.empty(t32.shape, dtype=torch.long, device=t32.device)
    _lib.check(_lib.lib().ocnn_table_to_i64(_lib.ptr(t32), t32.numel(), _lib.ptr(out),
                                            _lib.stream()))
    return out

  def get_neigh(self, depth: int, kernel: str = '333', stride: int = 1, nempty: bool = False):
    """int64 table (rows, K) with the reference's semantics
    (ocnn/octree/octree.py:490-523): the cached tensor itself for stride 1 (all
    nodes, or non-empty nodes with kernel '333'), a fresh tensor otherwise."""
    if stride not in (1, 2):
      raise ValueError('Unsupported stride {}'.format(stride))
    if kernel != '333' and kernel not in LUT_KERNEL:
      raise ValueError('Unsupported kernel {}'.format(kernel))
    if kernel == '333' and stride == 1:
      return self.nempty_neigh(depth) if nempty else self.neighs[depth]
    return self._widen(self._table(depth, kernel, stride, nempty))

  # ---- input signal (ocnn/octree/octree.py:525-568) -------------------------
  def get_input_feature(self, feature: str, nempty: bool = False):
    """The input signal of the finest layer, one block of channels per letter of `feature`, in
    the fixed order N D L P F whatever the order of the letters:
      N  the leaf normals (3)             D  <offset of the leaf's mean point from the
      L  that offset itself (3)              voxel centre, normal> (1)
      P  the mean point in [-1, 1] (3)    F  the leaf features
    Rows of empty nodes are zero unless nempty (ocnn/octree/octree.py:525-568)."""
    from ..nn.octree_pad import octree_pad
    depth, wanted = self.depth, set(feature.upper())
    normals, points = self.normals[depth], self.points[depth]
    offset = points.frac() - 0.5 if wanted & {'L', 'D'} else None
    blocks = {
        'N': lambda: normals,
        'D': lambda: (offset * normals).sum(dim=1, keepdim=True),
        'L': lambda: offset,
        'P': lambda: points * (2.0 ** (1 - depth)) - 1.0,
        'F': lambda: self.features[depth],
    }
    out = torch.cat([blocks[c]() for c in 'NDLPF' if c in wanted], dim=1)
    return out if nempty else octree_pad(out, self, depth)

  def to_points(self, rescale: bool = True):
    """The leaves as a point cloud: their mean points (voxel centres when the octree holds
    none), in [-1, 1] when rescale, with the leaf normals and features."""
    depth = self.depth
    xyz = self.points[depth]
    if xyz is None:
      x, y, z, batch_id = self.xyzb(depth, nempty=True)
      xyz = torch.stack([x, y, z], dim=1) + 0.5
    else:
      batch_id = self.batch_id(depth, nempty=True)
    if rescale:
      xyz = xyz * (2.0 ** (1 - depth)) - 1.0
    return Points(xyz, self.normals[depth], self.features[depth], batch_id=batch_id,
                  batch_size=self.batch_size)

  # ---- device moves, batching (ocnn/octree/octree.py:600-752) ---------------
  def to(self, device: Union[torch.device, str], non_blocking: bool = False):
    """A copy on `device` (the octree itself when it is there already).  The node counts are
    host tensors on any device, so that shape queries never wait for the GPU."""
    device = torch.device(device)
    if self.device == device:
      return self
    moved = Octree.init_like(self, device)
    for name in ('keys', 'children', 'features', 'normals', 'points'):
      setattr(moved, name, [None if t is None else t.to(device, non_blocking=non_blocking)
                            for t in getattr(self, name)])
    moved.neighs = self.neighs.moved(device, non_blocking)
    for name in ('nnum', 'nnum_nempty', 'batch_nnum', 'batch_nnum_nempty'):
      setattr(moved, name, getattr(self, name).clone())
    return moved

  def cuda(self, non_blocking: bool = False):
    return self.to('cuda', non_blocking)

  def cpu(self):
    return self.to('cpu')

  def merge_octrees(self, octrees: List['Octree']):
    """Batches single octrees (ocnn/octree/octree.py:653-717)."""
    bs = len(octrees)
    self.batch_size = bs
    for o in octrees[1:]:
      assert (o.depth == self.depth and o.full_depth == self.full_depth and
              o.device == self.device), 'The check of merge_octrees failed'
    batch_nnum = torch.stack([o.nnum for o in octrees], dim=1)
    batch_nnum_nempty = torch.stack([o.nnum_nempty for o in octrees], dim=1)
    self.nnum = torch.sum(batch_nnum, dim=1)
    self.nnum_nempty = torch.sum(batch_nnum_nempty, dim=1)
    self.batch_nnum = batch_nnum
    self.batch_nnum_nempty = batch_nnum_nempty
    offset = cumsum(batch_nnum_nempty, dim=1, exclusive=True)

    num = self.depth + 1
    self.neighs = _NeighTables(num)
    self.nempty_masks = [None] * num
    self.nempty_indices = [None] * num
    self.nempty_neighs = [None] * num
    self._nempty_indices32 = [None] * num
    self._tables, self._tables_t, self._plans = {}, {}, {}
    low48 = (1 << 48) - 1
    for d in range(num):
      self.keys[d] = torch.cat([(o.keys[d] & low48) | (i << 48)
                                for i, o in enumerate(octrees)], dim=0)
      kids = []
      for i, o in enumerate(octrees):
        c = o.children[d]
        kids.append(torch.where(c >= 0, c + int(offset[d, i]), c))
      self.children[d] = torch.cat(kids, dim=0)
      if d == self.depth:
        for name in ('features', 'normals', 'points'):
          if getattr(octrees[0], name)[d] is not None:
            getattr(self, name)[d] = torch.cat([getattr(o, name)[d] for o in octrees], dim=0)
    return self

  @classmethod
  def init_like(cls, octree: 'Octree', device: Union[torch.device, str, None] = None):
    device = device if device is not None else octree.device
    return cls(depth=octree.depth, full_depth=octree.full_depth,
               batch_size=octree.batch_size, device=device)

  @classmethod
  def init_octree(cls, depth: int, full_depth: int = 2, batch_size: int = 1,
                  device: Union[torch.device, str] = 'cpu'):
    octree = cls(depth, full_depth, batch_size, device)
    for d in range(full_depth + 1):
      octree.octree_grow_full(depth=d)
    return octree


def merge_octrees(octrees: List['Octree']):
  return Octree.init_like(octrees[0]).merge_octrees(octrees)


def init_octree(depth: int, full_depth: int = 2, batch_size: int = 1,
                device: Union[torch.device, str] = 'cpu'):
  return Octree.init_octree(depth, full_depth, batch_size, device)



Octree.plan_history = PlanHistory()
