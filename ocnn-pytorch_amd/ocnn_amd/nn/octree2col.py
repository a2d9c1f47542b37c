"""Explicit im2col form of the octree convolution (ocnn/nn/octree2col.py:15-53): the route
`method='explicit_gemm'` of OctreeConv / OctreeDeconv takes, kept as the slow, obviously
right counterpart of the gather-GEMM kernels.  Plain tensor indexing on the octree's device;
the scatter direction runs as a gather over the inverse table, so no atomics and a fixed
summation order here too."""

import torch

from .. import _lib
from ..octree.contract import tables_of


def octree2col(data: torch.Tensor, octree, depth: int, kernel_size: str = '333', stride: int = 1,
               nempty: bool = False):
  """(rows_in, C) -> (rows, K, C): entry (i, k) is the row of `data` that slot k of table row i
  names, zeros where it names none."""
  table = tables_of(octree)._table(depth, kernel_size, stride, nempty)
  _lib.require_gpu(data, table)
  hit = table >= 0
  col = data[table.clamp_min(0).long()]                  # (rows, K, C)
  return col * hit.unsqueeze(-1).to(data.dtype)


def col2octree(data: torch.Tensor, octree, depth: int, kernel_size: str = '333', stride: int = 1,
               nempty: bool = False):
  """(rows, K, C) -> (rows_in, C), the adjoint of octree2col: row j receives the sum of the
  entries (i, k) whose slot names j.  Every (j, k) has at most one such i (the inverse
  table), so the sum over k is taken in slot order."""
  rows_in = int(octree.nnum_nempty[depth] if nempty else octree.nnum[depth])
  inverse = tables_of(octree)._table_t(depth, kernel_size, stride, nempty, rows_in)     # (rows_in, K)
  _lib.require_gpu(data, inverse)
  K = inverse.shape[1]
  slot = torch.arange(K, device=data.device).expand_as(inverse)
  hit = inverse >= 0
  picked = data[inverse.clamp_min(0).long(), slot]       # (rows_in, K, C)
  return (picked * hit.unsqueeze(-1).to(data.dtype)).sum(1)
