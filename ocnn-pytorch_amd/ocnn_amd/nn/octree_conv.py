"""OctreeConv / OctreeDeconv with the module and functional API of the
reference (ocnn/nn/octree_conv.py), running on the HIP gather-GEMM and split-K
weight-gradient kernels.

Engine view.  With T the (rows, K) neighbour table of the layer:
  forward_gemm  : out[i]  = sum_k data[T[i,k]] @ W[k]            (gather)
  backward_gemm : gin[j] += sum_{T[i,k]=j} grad[i] @ W[k]^T      (scatter)
  weight_gemm   : gW[k]   = sum_i data[T[i,k]]^T (x) grad[i]
The scatter is run as a gather too: through the mirrored slot K-1-k when the
table is centrally symmetric (stride 1, every kernel but 2x2x2) and through
the inverse table otherwise, so no atomics are involved anywhere.
"""

import ctypes
from typing import List

import torch
import torch.nn.functional as F
import torch.nn
from torch.autograd import Function

from .. import _lib
from ..octree.contract import tables_of
from ..utils import list2str, resize_with_last_val, xavier_uniform_
from .octree2col import col2octree, octree2col
from .octree_pad import _depad_raw, _pad_raw, octree_depad, octree_pad


# (thresholds of the kernel selection live in the library, csrc/select.hip; these are the ones
# the layer level needs: when odd channel counts run zero-padded, and from how many rows on the
# pair-plan kernels pay for loading their weights)
PAD_MIN_ROWS = 16384
_CHOICES = {}            # kernel choices of the calls without a plan, by shape (see _conv_gather)
SPARSE_MAX_OCCUPANCY = 0.3
SPARSE_MIN_ROWS = 32768


# Stride 2 over all nodes, seen from the coarse side.  Row q of such a table is the first child
# of the non-empty coarse node q with its neighbours at the fine offsets delta in {-1, 0, 1}^3
# (ocnn/octree/octree.py:502-506).  The fine node at child c (bits x y z) of the coarse node q'
# is therefore named by the coarse nodes q = q' + e, e in {0, 1}^3 with e <= c per axis, in slot
# delta = c - 2 e: the data gradient of the fine rows, (parents, 8 children x channels) since
# the children of a non-empty node are eight consecutive rows, is a 2x2x2 stride-1 gather over the
# NON-EMPTY COARSE nodes (slots e, the octree's own '222' table) with block weights
# Wb[e][:, c] = W[slot(c - 2 e)]^T, zero where e > c.  That gather issues 8 x 8 blocks of
# matrix work per coarse row, of which 27 are real, where the gather over the inverse table
# (fine rows x all slots of the kernel) issues 8 x 27 for 27.
_BLOCK_MAPS = {}


def _block_map(kernel, device):
  """(index (64,), mask (8, 8, 1, 1)): the kernel's slot for (e, c), e and c as 4 x + 2 y + z."""
  key = (kernel, str(device))
  if key not in _BLOCK_MAPS:
    from ..octree.octree import LUT_KERNEL
    slots = list(range(27)) if kernel == '333' else LUT_KERNEL[kernel]
    m = torch.full((8, 8), -1, dtype=torch.long)
    for e in range(8):
      for c in range(8):
        d = [((c >> a) & 1) - 2 * ((e >> a) & 1) for a in (2, 1, 0)]
        k27 = 9 * (d[0] + 1) + 3 * (d[1] + 1) + (d[2] + 1)
        if min(d) >= -1 and k27 in slots:
          m[e, c] = slots.index(k27)
    m = m.to(device)
    _BLOCK_MAPS[key] = (m.clamp_min(0).view(-1), (m >= 0).view(8, 8, 1, 1))
  return _BLOCK_MAPS[key]



def conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias=None, plan=None, dense=False,
                in_index=None, pad_to=None):
  """out (rows, cout) = gather-GEMM over `table` (int32, (rows, K)).  With a
  tile plan of the same table (and a supported shape) the staged kernel runs.
  dense: the table is the one-slot identity (row i reads row i).
  in_index (int32, with dense only): row i reads row in_index[i] of `data`, which may then have
  more rows than the table (the compact rows of the non-empty nodes, read from a tensor over
  all nodes without a depad pass).
  pad_to = (octree, depth) (with dense only): the result comes back as octree_pad would make it,
  a row for every node of `depth`, zeros for the empty ones: the kernel writes its rows there."""
  if pad_to is not None:
    if not dense:
      return _pad_raw(conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, plan, dense, in_index),
                      *pad_to)
    return _conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, None, dense, in_index, pad_to)[0]
  out, planned = _conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, plan, dense, in_index)
  if planned and plan is not None and plan.overflow_rows is not None:
    # the few tiles that are too dense for the plan: plan-free kernel, results put in place
    sub, _ = _conv_gather(data, rows_in, plan.overflow_table, W, cout, transposed, reverse, bias, None, False)
    out.index_copy_(0, plan.overflow_rows, sub)
  return out


def _plan_args(plan):
  """(has_plan, max distinct rows, entries of the row lists, occupancy, reuse) for the
  selection functions of the library."""
  if plan is None:
    return 0, 0, 0, 1.0, 0.0
  return 1, plan.umax, plan.total, float(plan.occupancy), float(plan.reuse)


def _conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, plan, dense, in_index=None, pad_to=None):
  """conv_gather without the overflow rows of the plan; also returns whether a kernel on
  the plan ran.  The library picks the kernel (ocnn_conv_gather_choose)."""
  _lib.require_gpu(data, table, W)
  L = _lib.lib()
  data, W, table = data.contiguous(), W.contiguous(), table.contiguous()
  rows, K = table.shape
  cin = data.shape[1]
  assert W.dtype == data.dtype and table.dtype == torch.int32
  assert W.numel() == K * cin * cout, 'weights do not match the table and channels'
  if bias is not None:
    bias = bias.to(data.dtype).contiguous()
  code = _lib.dtype_code(data)
  # (the choice and the workspace size depend on the shapes and the plan only: asked once per plan)
  memo = _CHOICES if plan is None else plan.__dict__.setdefault('_choices', {})
  key = ('g', code, rows_in, rows, K, cin, cout, bool(dense))
  picked = memo.get(key)
  if picked is None:
    if len(memo) > 256:
      memo.clear()
    picked = memo[key] = (L.ocnn_conv_gather_choose(code, rows_in, rows, K, cin, cout, int(bool(dense)),
                                                     *_plan_args(plan)),
                          L.ocnn_conv_gather_workspace_bytes(code, rows_in, K, cin, cout))
  kernel, ws_bytes = picked
  if kernel == _lib.GATHER_DENSE_RW and (in_index is not None or pad_to is not None):
    # the indexed form also addresses the tensors over all nodes with 32-bit offsets: past that
    # range the rows are copied out (depad) / in (pad) around the kernel on the compact rows
    n_all = max(data.shape[0], rows if pad_to is None else int(pad_to[0].nnum[pad_to[1]]))
    if not L.ocnn_conv_dense_rw_supported(code, n_all, cin, cout):
      if in_index is not None:
        data, in_index = data.index_select(0, in_index.long()), None
      out, planned = _conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, plan, dense)
      return (out if pad_to is None else _pad_raw(out, *pad_to)), planned
  if in_index is not None and kernel != _lib.GATHER_DENSE_RW:
    data, in_index = data.index_select(0, in_index.long()), None       # the other kernels take compact rows
  if pad_to is not None and kernel != _lib.GATHER_DENSE_RW:          # the other kernels write compact rows
    out, planned = _conv_gather(data, rows_in, table, W, cout, transposed, reverse, bias, plan, dense, in_index)
    return _pad_raw(out, *pad_to), planned
  if kernel == _lib.GATHER_ZERO_PADDED:
    cin_p, cout_p = -(-cin // 32) * 32, -(-cout // 16) * 16
    Wk = W.view(K, cout, cin) if transposed else W.view(K, cin, cout)
    pad_w = (0, cin_p - cin, 0, cout_p - cout) if transposed else (0, cout_p - cout, 0, cin_p - cin)
    out = conv_gather(F.pad(data, (0, cin_p - cin)), rows_in, table, F.pad(Wk, pad_w), cout_p,
                      transposed, reverse, None if bias is None else F.pad(bias, (0, cout_p - cout)), plan)
    return out[:, :cout].contiguous(), False
  ws = _lib.workspace(ws_bytes, data.device)
  if kernel == _lib.GATHER_DENSE_RW:
    out_index, n_out = None, rows
    if pad_to is not None:
      octree, depth = pad_to
      out_index, n_out = octree._nempty_index32(depth), int(octree.nnum[depth])
      assert out_index.numel() == rows, 'conv_gather: one result row per non-empty node'
    out = torch.empty((n_out, cout), dtype=data.dtype, device=data.device)
    _lib.check(L.ocnn_conv_dense_rw_indexed(code, _lib.ptr(data), data.shape[0], _lib.ptr(in_index), rows,
                                            _lib.ptr(W), cin, cout, int(transposed), _lib.ptr(bias), _lib.ptr(out),
                                            n_out, _lib.ptr(out_index), _lib.ptr(ws), ws.numel(), _lib.stream()))
    if pad_to is not None:                                            # zeros for the empty nodes
      _lib.check(L.ocnn_pad(code, None, _lib.ptr(octree.children[depth]), n_out, cout, 0.0, _lib.ptr(out),
                            _lib.stream()))
    return out, False
  out = torch.empty((rows, cout), dtype=data.dtype, device=data.device)
  tail = (_lib.ptr(bias), _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream())
  if kernel == _lib.GATHER_DENSE:
    _lib.check(L.ocnn_conv_dense(code, _lib.ptr(data), rows, _lib.ptr(W), cin, cout, int(transposed), *tail))
    return out, False
  if kernel == _lib.GATHER_RW:
    _lib.check(L.ocnn_conv_gather_rw(
        code, _lib.ptr(data), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows),
        plan.umax, plan.total, rows, K, _lib.ptr(W), cin, cout, int(transposed), int(reverse), *tail))
    return out, True
  if kernel == _lib.GATHER_WIDE:
    _lib.check(L.ocnn_conv_gather_wide(
        code, _lib.ptr(data), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows),
        plan.umax, plan.total, float(plan.occupancy), rows, K, _lib.ptr(W), cin, cout, int(transposed),
        int(reverse), *tail))
    return out, True
  if kernel == _lib.GATHER_SPARSE:
    pp = plan.pairs()
    ws = _lib.workspace(L.ocnn_conv_gather_sparse_workspace_bytes(cin, cout), data.device)
    _lib.check(L.ocnn_conv_gather_sparse(
        code, _lib.ptr(data), rows_in, _lib.ptr(plan.uptr), _lib.ptr(plan.urows), plan.umax, plan.total,
        _lib.ptr(pp.cptr), _lib.ptr(pp.ent), pp.n_blocks, pp.max_blocks, _lib.ptr(pp.lists), pp.n_lists,
        ctypes.addressof(pp.group_bounds_host), rows, K, _lib.ptr(W), cin, cout, int(transposed), int(reverse),
        _lib.ptr(bias), _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
    return out, True
  if kernel == _lib.GATHER_PLANNED:
    _lib.check(L.ocnn_conv_gather_planned(
        code, _lib.ptr(data), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr),
        _lib.ptr(plan.urows), rows, K, _lib.ptr(W), cin, cout, int(transposed), int(reverse), *tail))
    return out, True
  _lib.check(L.ocnn_conv_gather(
      code, _lib.ptr(data), rows_in, _lib.ptr(table), rows, K, _lib.ptr(W),
      cin, cout, int(transposed), int(reverse), *tail))
  return out, False


def conv_wgrad(x, g, table, out_transposed=False, plan=None, dense=False, g_index=None):
  """gW (K, ca, cb) [or (K, cb, ca)] = sum_i x[T[i,k]]^T (x) g[i].  With a tile
  plan of the same table (and a supported shape) the staged kernel runs.
  dense: the table is the one-slot identity (row i reads row i).
  g_index (int32, with dense only): row i of the sum takes row g_index[i] of `g`, which may then
  have more rows than the table (see conv_gather)."""
  gw, planned = _conv_wgrad(x, g, table, out_transposed, plan, dense, g_index)
  if planned and plan is not None and plan.overflow_rows is not None:
    # the few tiles that are too dense for the plan: their share of the sums, plan-free kernel
    more, _ = _conv_wgrad(x, g.index_select(0, plan.overflow_rows), plan.overflow_table, out_transposed, None,
                          False)
    gw += more
  return gw


def _conv_wgrad(x, g, table, out_transposed, plan, dense, g_index=None):
  """conv_wgrad without the overflow rows of the plan; also returns whether a kernel on the
  plan ran.  The library picks the kernel (ocnn_conv_wgrad_choose)."""
  _lib.require_gpu(x, g, table)
  L = _lib.lib()
  x, g, table = x.contiguous(), g.contiguous(), table.contiguous()
  rows, K = table.shape
  ca, cb = x.shape[1], g.shape[1]
  code = _lib.dtype_code(x)
  memo = _CHOICES if plan is None else plan.__dict__.setdefault('_choices', {})
  key = ('w', code, x.shape[0], rows, K, ca, cb, bool(dense))
  kernel = memo.get(key)
  if kernel is None:
    if len(memo) > 256:
      memo.clear()
    kernel = memo[key] = L.ocnn_conv_wgrad_choose(code, x.shape[0], rows, K, ca, cb, int(bool(dense)),
                                                  *_plan_args(plan)[:4])
  if g_index is not None and (kernel != _lib.WGRAD_DENSE_RW or
                              not L.ocnn_conv_dense_wgrad_rw_supported(code, max(rows, g.shape[0]), ca, cb)):
    # (the other kernels take compact rows, and so does the dense one past its 32-bit offset range)
    g, g_index = g.index_select(0, g_index.long()), None
  assert (g_index is not None or g.shape[0] == rows) and x.dtype == g.dtype and table.dtype == torch.int32
  if kernel == _lib.WGRAD_ZERO_PADDED:
    ca_p, cb_p = -(-ca // 32) * 32, -(-cb // 32) * 32
    gw = conv_wgrad(F.pad(x, (0, ca_p - ca)), F.pad(g, (0, cb_p - cb)), table, out_transposed, plan)
    return (gw[:, :cb, :ca] if out_transposed else gw[:, :ca, :cb]).contiguous(), False
  shape = (K, cb, ca) if out_transposed else (K, ca, cb)
  gw = torch.empty(shape, dtype=x.dtype, device=x.device)
  if kernel == _lib.WGRAD_DENSE_RW:
    ws = _lib.workspace(L.ocnn_conv_dense_wgrad_rw_workspace_bytes(ca, cb), x.device)
    _lib.check(L.ocnn_conv_dense_wgrad_rw_indexed(code, _lib.ptr(x), x.shape[0], None, _lib.ptr(g), g.shape[0],
                                                  _lib.ptr(g_index), rows, ca, cb, int(out_transposed),
                                                  _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
    return gw, False
  if kernel == _lib.WGRAD_SPARSE:
    pp = plan.pairs()
    ws = _lib.workspace(L.ocnn_conv_wgrad_sparse_workspace_bytes(rows, ca, cb), x.device)
    _lib.check(L.ocnn_conv_wgrad_sparse(
        code, _lib.ptr(x), x.shape[0], ca, _lib.ptr(g), rows, cb, _lib.ptr(plan.uptr), _lib.ptr(plan.urows),
        plan.umax, plan.total, _lib.ptr(pp.cptr), _lib.ptr(pp.ent), pp.n_blocks,
        ctypes.addressof(pp.lists_host), ctypes.addressof(pp.list_count_host), pp.n_lists, K,
        int(not out_transposed), _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
    return gw, True
  if kernel == _lib.WGRAD_PLANNED:
    ws = _lib.workspace(L.ocnn_conv_wgrad_planned_workspace_bytes_for(code, x.shape[0], rows, K, ca, cb), x.device)
    _lib.check(L.ocnn_conv_wgrad_planned(
        code, _lib.ptr(x), x.shape[0], _lib.ptr(g), _lib.ptr(plan.loc), _lib.ptr(plan.uptr),
        _lib.ptr(plan.urows), plan.umax, plan.total, rows, K, ca, cb, int(out_transposed),
        _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
    return gw, True
  ws = _lib.workspace(L.ocnn_conv_wgrad_workspace_bytes_for(code, x.shape[0], rows, K, ca, cb), x.device)
  _lib.check(L.ocnn_conv_wgrad(
      code, _lib.ptr(x), x.shape[0], _lib.ptr(g), _lib.ptr(table), rows, K, ca, cb,
      int(out_transposed), _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
  return gw, False


def conv_wgrad_inverse(x, g, plan_t, out_transposed=False):
  """The same sums as conv_wgrad, taken over the INVERSE table (row j, slot k -> the row i
  with table[i][k] == j; plan_t is its tile plan): gW[k] = sum_j x[j]^T (x) g[Tt[j,k]].  For
  tables in which every row is pointed at from one slot only (2x2x2 stride 2: a node has one
  parent) the inverse has 1 / K of its entries set and tiles of few distinct rows, which is
  what the pair-plan kernel is made for.  None when the kernel does not take the shape."""
  _lib.require_gpu(x, g)
  L = _lib.lib()
  x, g = x.contiguous(), g.contiguous()
  K = plan_t.K
  cx, cg = x.shape[1], g.shape[1]
  code = _lib.DTYPE_CODE.get(x.dtype, -1)
  if not (plan_t.rows == x.shape[0] and plan_t.rows >= SPARSE_MIN_ROWS and
          plan_t.occupancy <= SPARSE_MAX_OCCUPANCY and x.dtype == g.dtype and
          L.ocnn_conv_wgrad_sparse_supported(code, g.shape[0], x.shape[0], K, cg, cx, plan_t.umax)):
    return None
  pp = plan_t.pairs()
  gw = torch.empty((K, cg, cx) if out_transposed else (K, cx, cg), dtype=x.dtype, device=x.device)
  ws = _lib.workspace(L.ocnn_conv_wgrad_sparse_workspace_bytes(x.shape[0], cg, cx), x.device)
  _lib.check(L.ocnn_conv_wgrad_sparse(
      code, _lib.ptr(g), g.shape[0], cg, _lib.ptr(x), x.shape[0], cx, _lib.ptr(plan_t.uptr),
      _lib.ptr(plan_t.urows), plan_t.umax, plan_t.total, _lib.ptr(pp.cptr), _lib.ptr(pp.ent), pp.n_blocks,
      ctypes.addressof(pp.lists_host), ctypes.addressof(pp.list_count_host), pp.n_lists, K, int(out_transposed),
      _lib.ptr(gw), _lib.ptr(ws), ws.numel(), _lib.stream()))
  if plan_t.overflow_rows is not None:                     # (tiles too dense for the plan)
    more, _ = _conv_wgrad(g, x.index_select(0, plan_t.overflow_rows), plan_t.overflow_table, not out_transposed,
                          None, False)
    gw += more
  return gw


def column_sum(g):
  """g.sum(0) with a fixed reduction order."""
  _lib.require_gpu(g)
  L = _lib.lib()
  g = g.contiguous()
  out = torch.empty(g.shape[1], dtype=g.dtype, device=g.device)
  ws = _lib.workspace(L.ocnn_colsum_workspace_bytes(g.shape[0], g.shape[1]), g.device)
  _lib.check(L.ocnn_colsum(_lib.dtype_code(g), _lib.ptr(g), g.shape[0], g.shape[1],
                           _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.stream()))
  return out


class OctreeConvBase:
  """Shapes and the three engine passes (ocnn/nn/octree_conv.py:26-202)."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False, max_buffer: int = int(2e8)):
    super().__init__()
    self.in_channels = in_channels
    self.out_channels = out_channels
    self.kernel_size = resize_with_last_val(kernel_size)
    self.kernel = list2str(self.kernel_size)
    self.stride = stride
    self.nempty = nempty
    self.max_buffer = max_buffer      # accepted for compatibility; nothing is buffered
    self.kdim = self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
    self.in_conv = in_channels if self.is_conv_layer() else out_channels
    self.out_conv = out_channels if self.is_conv_layer() else in_channels
    self.weights_shape = (self.kdim, self.in_conv, self.out_conv)

  def is_conv_layer(self):
    raise NotImplementedError

  def setup(self, octree, depth: int):
    """Heights of input/output and the table (ocnn/nn/octree_conv.py:51-100)."""
    # (an octree of another class gets its tables from its public members, octree/contract.py)
    octree = tables_of(octree)
    self.in_depth = self.out_depth = self.neigh_depth = depth
    if self.stride == 2:
      if self.is_conv_layer():
        self.out_depth = depth - 1
      else:
        self.out_depth = depth + 1
        self.neigh_depth = depth + 1
    if self.nempty:
      in_h = octree.nnum_nempty[self.in_depth]
      out_h = octree.nnum_nempty[self.out_depth]
    else:
      in_h = octree.nnum[self.in_depth]
      out_h = octree.nnum[self.out_depth]
      if self.stride == 2:
        if self.is_conv_layer():
          out_h = octree.nnum_nempty[self.out_depth]
        else:
          in_h = octree.nnum_nempty[self.in_depth]
    self.in_h, self.out_h = int(in_h), int(out_h)
    self.in_shape = (self.in_h, self.in_channels)
    self.out_shape = (self.out_h, self.out_channels)
    self.octree = octree
    self.neigh = octree._table(self.neigh_depth, self.kernel, self.stride, self.nempty)
    # rows on the "fine" side of the table (what its entries index)
    self.fine_h = self.in_h if self.is_conv_layer() else self.out_h
    self.symmetric = self.stride == 1 and self.kernel != '222'
    # 2x2x2 stride 2 over all nodes: row p of the table is exactly the 8 children 8p .. 8p+7
    # (children of a non-empty node are numbered consecutively, ocnn/octree/octree.py:235-259),
    # so the layer is a dense GEMM on the (P, 8 * C) view of the fine side: no gather at all
    self.dense_children = (self.kernel == '222' and self.stride == 2 and not self.nempty and
                           self.fine_h == 8 * self.neigh.shape[0])
    # the other kernels at stride 2 over all nodes: the data gradient in block form (_block_map)
    self.coarse_depth = self.out_depth if self.is_conv_layer() else self.in_depth
    self.block_children = (self.kernel != '222' and self.stride == 2 and not self.nempty and
                           self.fine_h == 8 * self.neigh.shape[0])

  def check_and_init(self, data: torch.Tensor):
    check = tuple(data.shape) == self.in_shape
    assert check, ('The shape of input data is wrong: ' +
                   'expected {}, got {}.'.format(self.in_shape, data.shape))

  def _inverse_table(self):
    return self.octree._table_t(self.neigh_depth, self.kernel, self.stride, self.nempty,
                                self.fine_h)

  def _plan(self, data, cin, cout, inverse=False):
    """Tile plan for the staged kernel, when the shape can use it."""
    L, code = _lib.lib(), _lib.DTYPE_CODE.get(data.dtype, -1)
    rows = data.shape[0]
    # (asked by every pass of every step: the answer is kept with the table it belongs to and
    # goes when the octree drops that table)
    memo = self.neigh.__dict__.setdefault('_plan_memo', {}) if hasattr(self.neigh, '__dict__') else None
    key = (code, rows, cin, cout, bool(inverse), self.fine_h)
    octree = self.octree
    ck = ((self.neigh_depth, self.kernel, self.stride, bool(self.nempty)), bool(inverse))
    if memo is not None and key in memo:
      plan = memo[key]
      if plan is None or octree._plans.get(ck) is plan:
        return plan
    if self.neigh.shape[0] >= PAD_MIN_ROWS:               # odd channel counts run zero-padded
      cin, cout = -(-cin // 32) * 32, -(-cout // 32) * 32
    if not (L.ocnn_conv_gather_planned_supported(code, rows, cin, cout) or
            L.ocnn_conv_gather_rw_supported(code, rows, self.kdim, cin, cout, 0) or
            L.ocnn_conv_gather_wide_supported(code, rows, self.kdim, cin, cout, 0) or
            L.ocnn_conv_gather_sparse_supported(code, rows, self.kdim, cin, cout, 0) or
            L.ocnn_conv_wgrad_planned_supported(code, rows, rows, self.kdim, cin, cout, 0)):
      plan = None
    else:
      plan = octree._plan(self.neigh_depth, self.kernel, self.stride, self.nempty, inverse, self.fine_h)
    if memo is not None:
      memo[key] = plan
    return plan

  def _identity(self, rows, device):
    """(rows, 1) table [0, 1, ..]: the one-slot 'gather' of the dense form."""
    cache = self.octree.__dict__.setdefault('_identity_tables', {})
    key = (rows, str(device))
    if key not in cache:
      cache[key] = torch.arange(rows, dtype=torch.int32, device=device).view(rows, 1)
    return cache[key]

  def forward_gemm(self, data, weights, bias=None, pad_to=None):
    """(fine rows, in_conv) -> (table rows, out_conv).  pad_to = (octree, depth): the result
    padded to all nodes of `depth` (octree_pad of the table rows)."""
    if self.dense_children:
      P = self.neigh.shape[0]
      return conv_gather(data.view(P, 8 * self.in_conv), P, self._identity(P, data.device),
                         weights.view(1, 8 * self.in_conv, self.out_conv), self.out_conv, False,
                         False, bias, None, dense=True, pad_to=pad_to)
    plan = self._plan(data, self.in_conv, self.out_conv)
    out = conv_gather(data, self.fine_h, self.neigh, weights, self.out_conv, False, False, bias,
                      plan)
    return out if pad_to is None else _pad_raw(out, *pad_to)

  def backward_gemm(self, grad, weights, bias=None, coarse_index=None):
    """(table rows, out_conv) -> (fine rows, in_conv).  coarse_index (int32): `grad` holds the
    table's rows at these rows of a larger tensor (all nodes of the depth, not only the
    non-empty ones the table has rows for)."""
    if self.dense_children:
      # gin.view(P, 8 * in_conv) = grad @ W'^T with W' = weights.view(8 * in_conv, out_conv)
      P = self.neigh.shape[0]
      b8 = None if bias is None else bias.repeat(8)
      out = conv_gather(grad, P, self._identity(P, grad.device),
                        weights.view(1, 8 * self.in_conv, self.out_conv), 8 * self.in_conv, True,
                        False, b8, None, dense=True, in_index=coarse_index)
      return out.view(8 * P, self.in_conv)
    if coarse_index is not None:
      grad = grad.index_select(0, coarse_index.long())
    if self.block_children:
      out = self._backward_blocks(grad, weights, bias)
      if out is not None:
        return out
    if self.symmetric:
      plan = self._plan(grad, self.out_conv, self.in_conv)
      return conv_gather(grad, grad.shape[0], self.neigh, weights, self.in_conv, True, True, bias,
                         plan)
    plan = self._plan(grad, self.out_conv, self.in_conv, inverse=True)
    return conv_gather(grad, grad.shape[0], self._inverse_table(), weights, self.in_conv, True,
                       False, bias, plan)

  def _backward_blocks(self, grad, weights, bias):
    """backward_gemm of a stride-2 layer over all nodes as a 2x2x2 stride-1 gather over the
    non-empty coarse nodes into the (parents, 8 x in_conv) view of the fine rows (_block_map).
    None where the kernels for wide layers do not take the shape (the caller then goes over
    the inverse table)."""
    L, code = _lib.lib(), _lib.DTYPE_CODE.get(grad.dtype, -1)
    P, wide = self.neigh.shape[0], 8 * self.in_conv
    octree = self.octree
    plan = octree._plan(self.coarse_depth, '222', 1, True)
    if L.ocnn_conv_gather_choose(code, P, P, 8, self.out_conv, wide, 0, *_plan_args(plan)) != _lib.GATHER_WIDE:
      return None
    index, valid = _block_map(self.kernel, grad.device)
    blocks = weights.view(self.kdim, self.in_conv, self.out_conv).index_select(0, index)
    blocks = blocks.view(8, 8, self.in_conv, self.out_conv) * valid.to(weights.dtype)          # e, c, in, out
    blocks = blocks.permute(0, 3, 1, 2).reshape(8, self.out_conv, wide)                        # e, out, (c, in)
    out = conv_gather(grad, P, octree._table(self.coarse_depth, '222', 1, True), blocks, wide, False, False,
                      None if bias is None else bias.repeat(8), plan)
    return out.view(8 * P, self.in_conv)

  def _weight_blocks(self, data, grad, out_transposed):
    """weight_gemm of a stride-2 layer over all nodes on the planned kernel: the fine rows as
    (parents, 8 x in_conv), the table of the eight coarse nodes whose children a row's slots
    reach (offsets {-1, 0}^3: slot delta of coarse node q reads child c = delta mod 2 of the node
    at e = floor(delta / 2)), sums (8, 8 x in_conv, out_conv) of which the kernel's slots are 27
    blocks at most.  None where the planned kernel does not take the shape."""
    L, code = _lib.lib(), _lib.DTYPE_CODE.get(data.dtype, -1)
    P, wide = self.neigh.shape[0], 8 * self.in_conv
    octree = self.octree
    plan = octree._plan(self.coarse_depth, '222m', 1, True)
    if L.ocnn_conv_wgrad_choose(code, P, P, 8, wide, self.out_conv, 0, *_plan_args(plan)[:4]) != _lib.WGRAD_PLANNED:
      return None
    sums = conv_wgrad(data.view(P, wide), grad, octree._table(self.coarse_depth, '222m', 1, True), False, plan)
    key = ('w', self.kernel, str(data.device))
    if key not in _BLOCK_MAPS:
      from ..octree.octree import LUT_KERNEL
      slots = list(range(27)) if self.kernel == '333' else LUT_KERNEL[self.kernel]
      e, c = [], []
      for k27 in slots:
        d = [k27 // 9 - 1, (k27 // 3) % 3 - 1, k27 % 3 - 1]
        e.append(sum((0 if v == -1 else 1) << (2 - a) for a, v in enumerate(d)))      # '222m' slot: offsets -1 -> 0, 0 -> 1
        c.append(sum((v & 1) << (2 - a) for a, v in enumerate(d)))                    # child bit: 1 for delta = +-1
      _BLOCK_MAPS[key] = (torch.tensor(e, device=data.device), torch.tensor(c, device=data.device))
    e, c = _BLOCK_MAPS[key]
    gw = sums.view(8, 8, self.in_conv, self.out_conv)[e, c]                             # (K, in_conv, out_conv)
    return gw.transpose(1, 2).contiguous() if out_transposed else gw

  def weight_gemm(self, data, grad, out_transposed=False, coarse_index=None):
    """data: fine rows; grad: table rows -> (K, in_conv, out_conv).  coarse_index: as in
    backward_gemm."""
    if self.dense_children:
      P = self.neigh.shape[0]
      gw = conv_wgrad(data.view(P, 8 * self.in_conv), grad, self._identity(P, data.device), False,
                      None, dense=True, g_index=coarse_index).view(8, self.in_conv, self.out_conv)
      return gw.transpose(1, 2).contiguous() if out_transposed else gw
    if coarse_index is not None:
      grad = grad.index_select(0, coarse_index.long())
    if self.block_children and self.kernel == '333':      # (8 x 8 blocks issued: a loss for 3 or 9 slots)
      gw = self._weight_blocks(data, grad, out_transposed)
      if gw is not None:
        return gw
    # (3x3x3 over all nodes: 20 of the 27 slots of a table row are set, and the plan-free kernel
    # over the table is faster than the pairs of the inverse)
    if self.stride == 2 and (self.kernel == '222' or (self.kernel == '333' and self.nempty)) and \
        self.neigh.shape[0] >= SPARSE_MIN_ROWS // 8 and \
        _lib.lib().ocnn_conv_wgrad_sparse_supported(_lib.DTYPE_CODE.get(data.dtype, -1), grad.shape[0],
                                                    data.shape[0], self.kdim, grad.shape[1], data.shape[1], 0):
      plan_t = self.octree._plan(self.neigh_depth, self.kernel, self.stride, self.nempty, True, self.fine_h)
      gw = conv_wgrad_inverse(data, grad, plan_t, out_transposed)
      if gw is not None:
        return gw
    plan = self._plan(data, self.in_conv, self.out_conv)
    return conv_wgrad(data, grad, self.neigh, out_transposed, plan)


class _OctreeConv(OctreeConvBase):
  def is_conv_layer(self): return True


class _OctreeDeconv(OctreeConvBase):
  def is_conv_layer(self): return False


class OctreeConvFunction(Function):
  """Autograd wiring of the convolution (ocnn/nn/octree_conv.py:219-254).  `bias` (optional)
  is added in the epilogue of the gather-GEMM kernel instead of by a pass of its own; its
  gradient is the fixed-order column sum of the output gradient.  `padded` (stride 2 over all
  nodes): the result comes back padded to all nodes of depth - 1 (what the module's octree_pad
  does, ocnn/nn/octree_conv.py:388-389), and the backward pass reads the rows of the non-empty
  nodes straight from the padded gradient through the octree's index of them: no depad pass."""

  @staticmethod
  def forward(ctx, data, weights, octree, depth: int, in_channels: int, out_channels: int,
              kernel_size: List[int] = [3, 3, 3], stride: int = 1, nempty: bool = False,
              max_buffer: int = int(2e8), bias=None, padded: bool = False):
    eng = _OctreeConv(in_channels, out_channels, kernel_size, stride, nempty, max_buffer)
    eng.setup(octree, depth)
    octree = eng.octree
    eng.check_and_init(data)
    data = data.contiguous()
    weights = weights.to(data.dtype).contiguous()
    out = eng.forward_gemm(data, weights, bias, pad_to=(octree, depth - 1) if padded else None)
    ctx.save_for_backward(data, weights)
    ctx.eng = eng
    ctx.pad_depth = depth - 1 if padded else None
    return out

  @staticmethod
  def backward(ctx, grad):
    data, weights = ctx.saved_tensors
    eng = ctx.eng
    grad = grad.contiguous()
    index = None
    if ctx.pad_depth is not None:
      if eng.dense_children and not ctx.needs_input_grad[10]:
        index = eng.octree._nempty_index32(ctx.pad_depth)       # the dense kernels read through it
      else:
        grad = _depad_raw(grad, eng.octree, ctx.pad_depth)      # one copy for all three gradients
    grad_out = eng.backward_gemm(grad, weights, coarse_index=index) if ctx.needs_input_grad[0] else None
    grad_w = eng.weight_gemm(data, grad, coarse_index=index) if ctx.needs_input_grad[1] else None
    grad_b = column_sum(grad) if ctx.needs_input_grad[10] else None
    return (grad_out, grad_w) + (None,) * 8 + (grad_b, None)


class OctreeDeconvFunction(Function):
  """Autograd wiring of the deconvolution (ocnn/nn/octree_conv.py:257-292).  `padded` (stride 2
  over all nodes): `data` has a row for every node of `depth` and the rows of the non-empty
  ones are read through the octree's index of them (what the module's octree_depad would copy
  out first, ocnn/nn/octree_conv.py:450-451); the data gradient comes back padded."""

  @staticmethod
  def forward(ctx, data, weights, octree, depth: int, in_channels: int, out_channels: int,
              kernel_size: List[int] = [3, 3, 3], stride: int = 1, nempty: bool = False,
              max_buffer: int = int(2e8), bias=None, padded: bool = False):
    eng = _OctreeDeconv(in_channels, out_channels, kernel_size, stride, nempty, max_buffer)
    eng.setup(octree, depth)
    octree = eng.octree
    index = None
    data = data.contiguous()
    if padded:
      assert tuple(data.shape) == (int(octree.nnum[depth]), in_channels), 'The shape of input data is wrong'
      if eng.dense_children:
        index = octree._nempty_index32(depth)                   # the dense kernels read through it
      else:
        data = _depad_raw(data, octree, depth)                  # one copy for forward and weight gradient
    else:
      eng.check_and_init(data)
    weights = weights.to(data.dtype).contiguous()
    out = eng.backward_gemm(data, weights, bias, coarse_index=index)
    ctx.save_for_backward(data, weights)
    ctx.eng = eng
    ctx.pad_depth = depth if padded else None
    ctx.indexed = index is not None
    return out

  @staticmethod
  def backward(ctx, grad):
    data, weights = ctx.saved_tensors
    eng = ctx.eng
    grad = grad.contiguous()
    index = eng.octree._nempty_index32(ctx.pad_depth) if ctx.indexed else None
    grad_out = None
    if ctx.needs_input_grad[0]:
      grad_out = eng.forward_gemm(grad, weights,
                                  pad_to=None if ctx.pad_depth is None else (eng.octree, ctx.pad_depth))
    # weights are (K, out_channels, in_channels): x = grad (fine side), g = data
    grad_w = eng.weight_gemm(grad, data, coarse_index=index) if ctx.needs_input_grad[1] else None
    grad_b = column_sum(grad) if ctx.needs_input_grad[10] else None
    return (grad_out, grad_w) + (None,) * 8 + (grad_b, None)


def octree_conv(data, weights, octree, depth: int, in_channels: int, out_channels: int,
                kernel_size: List[int] = [3, 3, 3], stride: int = 1, nempty: bool = False,
                max_buffer: int = int(2e8), bias=None, padded: bool = False):
  """Functional form (ocnn/nn/octree_conv.py:296), with an optional bias that the kernel adds
  and, for stride 2 over all nodes, the octree_pad of the result folded in (`padded`)."""
  return OctreeConvFunction.apply(data, weights, octree, depth, in_channels, out_channels, kernel_size, stride,
                                  nempty, max_buffer, bias, padded)


def octree_deconv(data, weights, octree, depth: int, in_channels: int, out_channels: int,
                  kernel_size: List[int] = [3, 3, 3], stride: int = 1, nempty: bool = False,
                  max_buffer: int = int(2e8), bias=None, padded: bool = False):
  """Functional form (ocnn/nn/octree_conv.py:297), with an optional bias that the kernel adds
  and, for stride 2 over all nodes, the octree_depad of the input folded in (`padded`)."""
  return OctreeDeconvFunction.apply(data, weights, octree, depth, in_channels, out_channels, kernel_size, stride,
                                    nempty, max_buffer, bias, padded)


class OctreeConv(OctreeConvBase, torch.nn.Module):
  """Octree convolution.  Constructor, parameters (`weights` (kdim, Cin, Cout),
  `bias`) and forward(data, octree, depth) follow ocnn/nn/octree_conv.py:300-431.
  `max_buffer` is accepted and ignored (nothing is buffered).  method='explicit_gemm' takes
  the reference's im2col route (octree2col + torch.mm, ocnn/nn/octree_conv.py:366-376); every
  other method name of the reference ('block_gemm', 'triton') and 'hip' run the HIP engine,
  for every kernel shape, stride and nempty mode."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False, method: str = 'triton',
               use_bias: bool = False, max_buffer: int = int(2e8)):
    super().__init__(in_channels, out_channels, kernel_size, stride, nempty, max_buffer)
    self.use_bias = use_bias
    self.method = self.check_method(method)
    self.weights = torch.nn.Parameter(torch.Tensor(*self.weights_shape))
    self.bias = torch.nn.Parameter(torch.Tensor(out_channels)) if use_bias else None
    self.reset_parameters()

  def check_method(self, method: str):
    if method not in ('explicit_gemm', 'block_gemm', 'triton', 'hip'):
      raise ValueError('Unknown method: {}'.format(method))
    return 'explicit_gemm' if method == 'explicit_gemm' else 'hip'

  def explicit_gemm(self, data: torch.Tensor, octree, depth: int):
    """im2col, then one matrix product (autograd differentiates the torch ops)."""
    col = octree2col(data, tables_of(octree), depth, self.kernel, self.stride, self.nempty)
    return torch.mm(col.flatten(1), self.weights.to(data.dtype).flatten(0, 1))

  def reset_parameters(self):
    xavier_uniform_(self.weights)
    if self.use_bias:
      torch.nn.init.zeros_(self.bias)

  def is_conv_layer(self): return True

  def forward(self, data: torch.Tensor, octree, depth: int):
    pad = self.stride == 2 and not self.nempty
    if self.method == 'explicit_gemm':
      out = self.explicit_gemm(data, octree, depth)
    else:
      # bias: in the kernel's epilogue; the pad: inside the function, whose backward pass then
      # needs no depad
      return octree_conv(data, self.weights, octree, depth, self.in_channels, self.out_channels,
                         self.kernel_size, self.stride, self.nempty, self.max_buffer,
                         self.bias if self.use_bias else None, pad)
    if self.use_bias:
      out = out + self.bias.to(out.dtype)
    if pad:
      out = octree_pad(out, octree, depth - 1)
    return out

  def extra_repr(self) -> str:
    return ('in_channels={}, out_channels={}, kernel_size={}, stride={}, '
            'nempty={}, bias={}, method={}').format(
                self.in_channels, self.out_channels, self.kernel_size, self.stride,
                self.nempty, self.use_bias, self.method)


class OctreeDeconv(OctreeConv):
  """Octree deconvolution (ocnn/nn/octree_conv.py:433-466); weights are
  (kdim, out_channels, in_channels)."""

  def is_conv_layer(self): return False

  def forward(self, data: torch.Tensor, octree, depth: int):
    depad = self.stride == 2 and not self.nempty
    if self.method != 'explicit_gemm':
      # the depad: inside the function, which reads the rows of the non-empty nodes through an index
      return octree_deconv(data, self.weights, octree, depth, self.in_channels, self.out_channels,
                           self.kernel_size, self.stride, self.nempty, self.max_buffer,
                           self.bias if self.use_bias else None, depad)
    if depad:
      data = octree_depad(data, octree, depth)
    if self.method == 'explicit_gemm':
      # one product for all slots, then the adjoint of im2col (ocnn/nn/octree_conv.py:453-457)
      col = torch.mm(data, self.weights.to(data.dtype).flatten(0, 1).t())
      out = col2octree(col.view(col.shape[0], self.kdim, -1), tables_of(octree), depth + (self.stride == 2), self.kernel,
                       self.stride, self.nempty)
    else:
      out = octree_deconv(data, self.weights, octree, depth, self.in_channels, self.out_channels,
                          self.kernel_size, self.stride, self.nempty, self.max_buffer,
                          self.bias if self.use_bias else None)
    if self.use_bias and self.method == 'explicit_gemm':
      out = out + self.bias.to(out.dtype)
    return out
