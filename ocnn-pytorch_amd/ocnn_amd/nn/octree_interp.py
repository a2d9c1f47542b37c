"""Point interpolation and upsampling with the API of ocnn/nn/octree_interp.py on HIP
kernels: the neighbour search and the weights in one kernel, the weighted row gather (and
its transpose for the gradient) in another.  No atomics: the gradient with respect to the
data runs over the transposed sparse matrix in row form."""

from typing import Optional, Union

import torch
import torch.nn

from .. import _lib
from .octree_pad import octree_depad


def _csr_rows(data, col, val, rowptr, kfixed, rowdiv, rows):
  out = torch.empty((rows, data.shape[1]), dtype=data.dtype, device=data.device)
  _lib.check(_lib.lib().ocnn_csr_rows(_lib.dtype_code(data), _lib.ptr(rowptr), kfixed, _lib.ptr(col),
                                      _lib.ptr(val), _lib.ptr(data), data.shape[1], _lib.ptr(rowdiv),
                                      _lib.ptr(out), rows, _lib.stream()))
  return out


def _transpose(idx, w, norm, rows):
  """Row form of the transposed matrix of (point, neighbour) entries: for every data row the
  points that read it (ascending) and their weights, divided by the points' weight sums."""
  L = _lib.lib()
  m, k = idx.shape
  ws = _lib.workspace(L.ocnn_csr_transpose_workspace_bytes(m * k), idx.device)
  rowptr = torch.empty(rows + 1, dtype=torch.int32, device=idx.device)
  col = torch.empty(m * k, dtype=torch.int32, device=idx.device)
  val = None if w is None and norm is None else torch.empty(m * k, dtype=torch.float32, device=idx.device)
  _lib.check(L.ocnn_csr_transpose(_lib.ptr(idx), _lib.ptr(w), _lib.ptr(norm), m, k, rows, _lib.ptr(ws),
                                  ws.numel(), _lib.ptr(rowptr), _lib.ptr(col), _lib.ptr(val), _lib.stream()))
  return rowptr, col, val


class _Interp(torch.autograd.Function):
  """out[p] = (sum_j w[p, j] data[idx[p, j]]) / (norm[p] + 1e-12)   (norm None: no division)."""

  @staticmethod
  def forward(ctx, data, idx, w, norm):
    data = data.contiguous()
    ctx.save_for_backward(idx, w, norm)
    ctx.rows = data.shape[0]
    return _csr_rows(data, idx, w, None, idx.shape[1], norm, idx.shape[0])

  @staticmethod
  def backward(ctx, grad):
    idx, w, norm = ctx.saved_tensors
    rowptr, col, val = _transpose(idx, w, norm, ctx.rows)
    return _csr_rows(grad.contiguous(), col, val, rowptr, 0, None, ctx.rows), None, None, None


def _keys(octree, depth, nempty):
  return octree.key(depth, nempty).contiguous()


def _tree(octree, depth, nempty):
  """Arguments of the library's walks down the tree (host array of the children arrays, depth,
  full depth, batch size, nempty), or None where an array is missing or not on the device."""
  import ctypes
  top = min(depth, octree.full_depth)
  need = range(top, depth + 1 if nempty else depth)
  if any(octree.children[l] is None or not octree.children[l].is_cuda for l in need):
    return None
  ptrs = [None if octree.children[l] is None else octree.children[l].data_ptr() for l in range(depth + 1)]
  return (ctypes.c_void_p * (depth + 1))(*ptrs), depth, octree.full_depth, octree.batch_size, int(bool(nempty))


def _pts(pts):
  _lib.require_gpu(pts)
  assert pts.dim() == 2 and pts.shape[1] == 4, 'pts: (N, 4) rows of (x, y, z, batch)'
  return pts.to(torch.float32).contiguous()


def _check_rows(data, octree, depth, nempty):
  nnum = octree.nnum_nempty[depth] if nempty else octree.nnum[depth]
  assert data.shape[0] == nnum, 'The shape of input data is wrong.'


def octree_nearest_pts(data: torch.Tensor, octree, depth: int, pts: torch.Tensor,
                       nempty: bool = False, bound_check: bool = False):
  """Nearest-neighbour interpolation at points scaled to [0, 2^depth)
  (ocnn/nn/octree_interp.py:15-46): the row of the node that holds the point, zeros where
  there is none."""
  _check_rows(data, octree, depth, nempty)
  pts = _pts(pts)
  idx = torch.empty((pts.shape[0], 1), dtype=torch.int32, device=pts.device)
  tree = _tree(octree, depth, nempty)
  if tree is not None:
    _lib.check(_lib.lib().ocnn_locate_points(_lib.ptr(pts), pts.shape[0], *tree, int(bound_check), _lib.ptr(idx),
                                             _lib.stream()))
  else:
    keys = _keys(octree, depth, nempty)
    _lib.check(_lib.lib().ocnn_search_points(_lib.ptr(pts), pts.shape[0], depth, _lib.ptr(keys),
                                             keys.numel(), int(bound_check), _lib.ptr(idx), _lib.stream()))
  return _Interp.apply(data, idx, None, None)


def octree_linear_pts(data: torch.Tensor, octree, depth: int, pts: torch.Tensor,
                      nempty: bool = False, bound_check: bool = False):
  """Trilinear interpolation over the (up to 8) existing neighbours, normalised by their
  weight sum (ocnn/nn/octree_interp.py:49-103)."""
  _check_rows(data, octree, depth, nempty)
  pts = _pts(pts)
  m = pts.shape[0]
  idx = torch.empty((m, 8), dtype=torch.int32, device=pts.device)
  w = torch.empty((m, 8), dtype=torch.float32, device=pts.device)
  norm = torch.empty(m, dtype=torch.float32, device=pts.device)
  tree = _tree(octree, depth, nempty)
  if tree is not None:
    _lib.check(_lib.lib().ocnn_interp_linear_locate(_lib.ptr(pts), m, *tree, int(bound_check), _lib.ptr(idx),
                                                    _lib.ptr(w), _lib.ptr(norm), _lib.stream()))
  else:
    keys = _keys(octree, depth, nempty)
    _lib.check(_lib.lib().ocnn_interp_linear_prepare(_lib.ptr(pts), m, depth, _lib.ptr(keys), keys.numel(),
                                                     int(bound_check), _lib.ptr(idx), _lib.ptr(w),
                                                     _lib.ptr(norm), _lib.stream()))
  return _Interp.apply(data, idx, w, norm)


class OctreeInterp(torch.nn.Module):
  """ocnn/nn/octree_interp.py:106-141."""

  def __init__(self, method: str = 'linear', nempty: bool = False, bound_check: bool = False,
               rescale_pts: bool = True):
    super().__init__()
    self.method = method
    self.nempty = nempty
    self.bound_check = bound_check
    self.rescale_pts = rescale_pts
    self.func = octree_linear_pts if method == 'linear' else octree_nearest_pts

  def forward(self, data: torch.Tensor, octree, depth: int, pts: torch.Tensor,
              bbmin: Union[torch.Tensor, float] = -1, bbmax: Union[torch.Tensor, float] = 1):
    # points from [bbmin, bbmax] to [0, 2^depth], in place like the reference
    if self.rescale_pts:
      box_size = bbmax - bbmin
      if type(box_size) is torch.Tensor:
        box_size = box_size.max().item()
      assert box_size > 0, 'The bounding box size must be greater than 0.'
      pts[:, :3] = (pts[:, :3] - bbmin) * (2 ** depth / box_size)
    return self.func(data, octree, depth, pts, self.nempty, self.bound_check)

  def extra_repr(self) -> str:
    return 'method={}, nempty={}, bound_check={}, rescale_pts={}'.format(
        self.method, self.nempty, self.bound_check, self.rescale_pts)


def octree_nearest_upsample(data: torch.Tensor, octree, depth: int, nempty: bool = False):
  """depth -> depth + 1, every child takes its parent's row (ocnn/nn/octree_interp.py:144-167)."""
  _check_rows(data, octree, depth, nempty)
  out = data
  if not nempty:
    out = octree_depad(out, octree, depth)
  out = out.unsqueeze(1).repeat(1, 8, 1).flatten(end_dim=1)
  if nempty:
    out = octree_depad(out, octree, depth + 1)
  return out


class OctreeUpsample(torch.nn.Module):
  """depth -> target_depth (ocnn/nn/octree_interp.py:170-200)."""

  def __init__(self, method: str = 'linear', nempty: bool = False):
    super().__init__()
    self.method = method
    self.nempty = nempty
    self.func = octree_linear_pts if method == 'linear' else octree_nearest_pts

  def forward(self, data: torch.Tensor, octree, depth: int, target_depth: Optional[int] = None):
    if target_depth is None:
      target_depth = depth + 1
    if target_depth == depth:
      return data
    assert target_depth >= depth, 'target_depth must be larger than depth'
    if target_depth == depth + 1 and self.method == 'nearest':
      return octree_nearest_upsample(data, octree, depth, self.nempty)
    xyzb = octree.xyzb(target_depth, self.nempty)
    pts = torch.stack(xyzb, dim=1).float()
    pts[:, :3] = (pts[:, :3] + 0.5) * (2 ** (depth - target_depth))
    return self.func(data, octree, depth, pts, self.nempty)

  def extra_repr(self) -> str:
    return 'method={}, nempty={}'.format(self.method, self.nempty)
