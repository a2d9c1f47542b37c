"""Pooling with the API of ocnn/nn/octree_pool.py on HIP kernels: 2x2x2 max pooling /
unpooling, average pooling over a neighbour table, global average pooling per batch element."""

from typing import List

import torch
import torch.nn

from .. import _lib
from ..octree.contract import tables_of
from ..utils import list2str, resize_with_last_val
from .octree_pad import octree_pad


def _rows(octree, depth, nempty):
  return int(octree.nnum_nempty[depth] if nempty else octree.nnum[depth])


def _pool_raw(data, octree, depth, nempty):
  """(rows at depth, C) -> (rows at depth - 1, C), indices (non-empty parents, C) int64."""
  _lib.require_gpu(data)
  data = data.contiguous()
  assert data.shape[0] == _rows(octree, depth, nempty), 'octree_max_pool: wrong number of rows'
  c = data.shape[1]
  parents = int(octree.nnum[depth]) // 8
  out_rows = parents if nempty else int(octree.nnum[depth - 1])
  out = torch.empty((out_rows, c), dtype=data.dtype, device=data.device)
  indices = torch.empty((parents, c), dtype=torch.long, device=data.device)
  fine = octree.children[depth] if nempty else None
  coarse = None if nempty else octree.children[depth - 1]
  _lib.check(_lib.lib().ocnn_max_pool(_lib.dtype_code(data), _lib.ptr(data), _lib.ptr(fine),
                                      _lib.ptr(coarse), out_rows, c, _lib.ptr(out),
                                      _lib.ptr(indices), _lib.stream()))
  return out, indices


def _unpool_raw(data, indices, octree, depth, nempty):
  """(rows at depth, C) -> (rows at depth + 1, C): every value to the child `indices` names."""
  _lib.require_gpu(data, indices)
  data, indices = data.contiguous(), indices.contiguous()
  assert data.shape[0] == _rows(octree, depth, nempty), 'octree_max_unpool: wrong number of rows'
  c = data.shape[1]
  assert indices.shape == (int(octree.nnum[depth + 1]) // 8, c) and indices.dtype == torch.long
  out_rows = _rows(octree, depth + 1, nempty)
  out = torch.empty((out_rows, c), dtype=data.dtype, device=data.device)
  # non-empty form: out row r is node nempty_index[r] of the fine level, source row = parent;
  # all-nodes form: out row = node, source row = the parent's node at the coarse level
  octree = tables_of(octree)
  out_node = octree._nempty_index32(depth + 1) if nempty else None
  src_row = None if nempty else octree._nempty_index32(depth)
  _lib.check(_lib.lib().ocnn_max_unpool(_lib.dtype_code(data), _lib.ptr(data), _lib.ptr(indices),
                                        _lib.ptr(out_node), _lib.ptr(src_row), out_rows, c,
                                        _lib.ptr(out), _lib.stream()))
  return out


def _gather_raw(grad, indices, octree, depth, nempty):
  """Gradient of _unpool_raw: (rows at depth + 1, C) -> (rows at depth, C)."""
  _lib.require_gpu(grad, indices)
  grad, indices = grad.contiguous(), indices.contiguous()
  c = grad.shape[1]
  parents = indices.shape[0]
  out = torch.empty((parents, c), dtype=grad.dtype, device=grad.device)
  fine = octree.children[depth + 1] if nempty else None
  _lib.check(_lib.lib().ocnn_max_gather(_lib.dtype_code(grad), _lib.ptr(grad), _lib.ptr(indices),
                                        _lib.ptr(fine), parents, c, _lib.ptr(out), _lib.stream()))
  return out if nempty else octree_pad(out, octree, depth)


class _MaxPool(torch.autograd.Function):
  @staticmethod
  def forward(ctx, data, octree, depth, nempty):
    out, indices = _pool_raw(data, octree, depth, nempty)
    ctx.octree, ctx.depth, ctx.nempty = octree, depth, nempty
    ctx.save_for_backward(indices)
    ctx.mark_non_differentiable(indices)
    return out, indices

  @staticmethod
  def backward(ctx, grad, _):
    indices, = ctx.saved_tensors
    return _unpool_raw(grad, indices, ctx.octree, ctx.depth - 1, ctx.nempty), None, None, None


class _MaxUnpool(torch.autograd.Function):
  @staticmethod
  def forward(ctx, data, indices, octree, depth, nempty):
    ctx.octree, ctx.depth, ctx.nempty = octree, depth, nempty
    ctx.save_for_backward(indices)
    return _unpool_raw(data, indices, octree, depth, nempty)

  @staticmethod
  def backward(ctx, grad):
    indices, = ctx.saved_tensors
    return _gather_raw(grad, indices, ctx.octree, ctx.depth, ctx.nempty), None, None, None, None


def octree_max_pool(data: torch.Tensor, octree, depth: int, nempty: bool = False,
                    return_indices: bool = False):
  """Max pooling with kernel 2 and stride 2 (ocnn/nn/octree_pool.py:16-37): depth ->
  depth - 1.  One fused kernel: the -inf padding of the non-empty form, the maximum over the
  8 children, and the zero padding of the all-nodes form."""
  out, indices = _MaxPool.apply(data, octree, depth, nempty)
  return (out, indices) if return_indices else out


def octree_max_unpool(data: torch.Tensor, indices: torch.Tensor, octree, depth: int,
                      nempty: bool = False):
  """Max unpooling (ocnn/nn/octree_pool.py:40-65): depth -> depth + 1."""
  return _MaxUnpool.apply(data, indices, octree, depth, nempty)


class OctreeMaxPool(torch.nn.Module):
  """ocnn/nn/octree_pool.py:143-156."""

  def __init__(self, nempty: bool = False, return_indices: bool = False):
    super().__init__()
    self.kernel_size, self.kernel, self.stride = [2, 2, 2], '222', 2
    self.nempty = nempty
    self.return_indices = return_indices

  def forward(self, data: torch.Tensor, octree, depth: int):
    return octree_max_pool(data, octree, depth, self.nempty, self.return_indices)

  def extra_repr(self) -> str:
    return 'kernel_size={}, stride={}, nempty={}'.format(self.kernel_size, self.stride, self.nempty)


class OctreeMaxUnpool(torch.nn.Module):
  """ocnn/nn/octree_pool.py:159-171."""

  def __init__(self, nempty: bool = False):
    super().__init__()
    self.kernel_size, self.kernel, self.stride = [2, 2, 2], '222', 2
    self.nempty = nempty

  def forward(self, data: torch.Tensor, indices: torch.Tensor, octree, depth: int):
    return octree_max_unpool(data, indices, octree, depth, self.nempty)

  def extra_repr(self) -> str:
    return 'kernel_size={}, stride={}, nempty={}'.format(self.kernel_size, self.stride, self.nempty)


def octree_avg_pool(data: torch.Tensor, octree, depth: int, kernel: str, stride: int = 2,
                    nempty: bool = False):
  """Average over the existing neighbours of the table (ocnn/nn/octree_pool.py:68-101): the
  row-gather kernel of the interpolation with unit weights, divided by the neighbour count;
  the gradient runs over the transposed table (no atomics)."""
  from .octree_interp import _Interp
  table = tables_of(octree)._table(depth, kernel, stride, nempty)
  count = (table >= 0).sum(1).to(torch.float32)
  return _Interp.apply(data, table, None, count)


class _GlobalPool(torch.autograd.Function):
  @staticmethod
  def forward(ctx, data, bounds, batch_id, batch_size):
    from .octree_conv import column_sum
    data = data.contiguous()
    out = torch.zeros((batch_size, data.shape[1]), dtype=data.dtype, device=data.device)
    counts = []
    for b in range(batch_size):
      lo, hi = bounds[b], bounds[b + 1]
      counts.append(max(hi - lo, 1))                    # (an element may have no node)
      if hi > lo:
        out[b] = (column_sum(data[lo:hi]).float() / counts[-1]).to(data.dtype)
    ctx.count = torch.tensor(counts, dtype=torch.float32, device=data.device)
    ctx.save_for_backward(batch_id)
    return out

  @staticmethod
  def backward(ctx, grad):
    batch_id, = ctx.saved_tensors
    g = (grad.float() / ctx.count.unsqueeze(1)).to(grad.dtype)
    return g.index_select(0, batch_id), None, None, None


def octree_global_pool(data: torch.Tensor, octree, depth: int, nempty: bool = False):
  """Mean over the nodes of every batch element (ocnn/nn/octree_pool.py:104-125).  The nodes of
  an element are consecutive rows (the batch index is the top of the key), so each mean is a
  column sum with a fixed reduction order."""
  batch_id = octree.batch_id(depth, nempty)
  batch_size = octree.batch_size
  edges = torch.searchsorted(batch_id, torch.arange(batch_size + 1, device=batch_id.device))
  return _GlobalPool.apply(data, edges.tolist(), batch_id, batch_size)


class OctreeAvgPool(torch.nn.Module):
  """ocnn/nn/octree_pool.py:190-200."""

  def __init__(self, kernel_size: List[int], stride: int, nempty: bool = False):
    super().__init__()
    self.kernel_size = resize_with_last_val(kernel_size)
    self.kernel = list2str(self.kernel_size)
    self.stride = stride
    self.nempty = nempty

  def forward(self, data: torch.Tensor, octree, depth: int):
    return octree_avg_pool(data, octree, depth, self.kernel, self.stride, self.nempty)

  def extra_repr(self) -> str:
    return 'kernel_size={}, stride={}, nempty={}'.format(self.kernel_size, self.stride, self.nempty)


class OctreeGlobalPool(torch.nn.Module):
  """ocnn/nn/octree_pool.py:174-187."""

  def __init__(self, nempty: bool = False):
    super().__init__()
    self.kernel_size, self.kernel, self.stride = [-1, -1, -1], '-1-1-1', -1
    self.nempty = nempty

  def forward(self, data: torch.Tensor, octree, depth: int):
    return octree_global_pool(data, octree, depth, self.nempty)

  def extra_repr(self) -> str:
    return 'kernel_size={}, stride={}, nempty={}'.format(self.kernel_size, self.stride, self.nempty)
