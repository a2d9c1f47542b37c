"""octree_pad / octree_depad (ocnn/nn/octree_pad.py) as HIP row scatters."""

import torch

from .. import _lib


def _children32(octree, depth):
  """children[depth] as the kernels read it: int32, contiguous (the reference's own dtype,
  ocnn/octree/octree.py:59; another integer type is converted)."""
  children = octree.children[depth]
  _lib.require_gpu(children)
  return children if children.dtype == torch.int32 and children.is_contiguous() else children.int().contiguous()


def _pad_raw(data: torch.Tensor, octree, depth: int, val: float = 0.0):
  children = _children32(octree, depth)
  _lib.require_gpu(data, children)
  data = data.contiguous()
  assert data.shape[0] == int(octree.nnum_nempty[depth]), 'octree_pad: wrong number of rows'
  n, c = int(octree.nnum[depth]), data.shape[1]
  out = torch.empty((n, c), dtype=data.dtype, device=data.device)
  _lib.check(_lib.lib().ocnn_pad(_lib.dtype_code(data), _lib.ptr(data), _lib.ptr(children), n, c,
                                 float(val), _lib.ptr(out), _lib.stream()))
  return out


def _depad_raw(data: torch.Tensor, octree, depth: int):
  children = _children32(octree, depth)
  _lib.require_gpu(data, children)
  data = data.contiguous()
  assert data.shape[0] == int(octree.nnum[depth]), 'octree_depad: wrong number of rows'
  n, c = data.shape[0], data.shape[1]
  out = torch.empty((int(octree.nnum_nempty[depth]), c), dtype=data.dtype, device=data.device)
  _lib.check(_lib.lib().ocnn_depad(_lib.dtype_code(data), _lib.ptr(data), _lib.ptr(children), n, c,
                                   _lib.ptr(out), _lib.stream()))
  return out


class _Pad(torch.autograd.Function):
  @staticmethod
  def forward(ctx, data, octree, depth, val):
    ctx.octree, ctx.depth = octree, depth
    return _pad_raw(data, octree, depth, val)

  @staticmethod
  def backward(ctx, grad):
    return _depad_raw(grad, ctx.octree, ctx.depth), None, None, None


class _Depad(torch.autograd.Function):
  @staticmethod
  def forward(ctx, data, octree, depth):
    ctx.octree, ctx.depth = octree, depth
    return _depad_raw(data, octree, depth)

  @staticmethod
  def backward(ctx, grad):
    return _pad_raw(grad, ctx.octree, ctx.depth, 0.0), None, None


def octree_pad(data: torch.Tensor, octree, depth: int, val: float = 0.0):
  """(nnum_nempty[depth], C) -> (nnum[depth], C); empty nodes get `val`.
  Differentiable.  Mirrors ocnn/nn/octree_pad.py:13-29."""
  return _Pad.apply(data, octree, depth, val)


def octree_depad(data: torch.Tensor, octree, depth: int):
  """(nnum[depth], C) -> (nnum_nempty[depth], C): rows of the non-empty nodes.
  Differentiable.  Mirrors ocnn/nn/octree_pad.py:32-39."""
  return _Depad.apply(data, octree, depth)
