"""OctreeDWConv with the API of ocnn/nn/octree_dwconv.py on HIP kernels."""

from typing import List

import torch
import torch.nn
from torch.autograd import Function

from .. import _lib
from ..utils import xavier_uniform_
from .octree_conv import OctreeConvBase
from .octree_pad import octree_pad


def dw_gather(data, rows_in, table, w, reverse, bias=None, plan=None):
  """out[i,c] = sum_k data[T[i,k],c] * w[k',c].  With a tile plan of the same table (and a
  supported shape) the kernel that stages a tile's rows in LDS runs."""
  _lib.require_gpu(data, table, w)
  L = _lib.lib()
  data, w, table = data.contiguous(), w.contiguous(), table.contiguous()
  rows, K = table.shape
  C = data.shape[1]
  assert w.numel() == K * C and w.dtype == data.dtype and table.dtype == torch.int32
  if bias is not None:
    bias = bias.to(data.dtype).contiguous()
  out = torch.empty((rows, C), dtype=data.dtype, device=data.device)
  code = _lib.DTYPE_CODE.get(data.dtype, -1)
  if plan is not None and plan.reuse >= 2.0 and L.ocnn_dwconv_gather_planned_supported(
      code, rows_in, K, C, plan.umax):
    _lib.check(L.ocnn_dwconv_gather_planned(
        code, _lib.ptr(data), rows_in, _lib.ptr(plan.loc), _lib.ptr(plan.uptr), _lib.ptr(plan.urows),
        plan.umax, plan.total, rows, K, _lib.ptr(w), C, int(reverse), _lib.ptr(bias), _lib.ptr(out),
        _lib.stream()))
    if plan.overflow_rows is not None:                     # the few tiles too dense for the plan
      out.index_copy_(0, plan.overflow_rows, dw_gather(data, rows_in, plan.overflow_table, w, reverse, bias))
    return out
  _lib.check(L.ocnn_dwconv_gather(
      _lib.dtype_code(data), _lib.ptr(data), rows_in, _lib.ptr(table), rows, K, _lib.ptr(w), C,
      int(reverse), _lib.ptr(bias), _lib.ptr(out), _lib.stream()))
  return out


def dw_wgrad(x, g, table, plan=None):
  """gw[k,0,c] = sum_i x[T[i,k],c] * g[i,c]."""
  _lib.require_gpu(x, g, table)
  L = _lib.lib()
  x, g, table = x.contiguous(), g.contiguous(), table.contiguous()
  rows, K = table.shape
  C = x.shape[1]
  assert g.shape == (rows, C) and x.dtype == g.dtype
  gw = torch.empty((K, 1, C), dtype=x.dtype, device=x.device)
  code = _lib.DTYPE_CODE.get(x.dtype, -1)
  if plan is not None and plan.reuse >= 2.0 and L.ocnn_dwconv_wgrad_planned_supported(
      code, x.shape[0], rows, K, C, plan.umax):
    ws = _lib.workspace(L.ocnn_dwconv_wgrad_planned_workspace_bytes(K, C), x.device)
    _lib.check(L.ocnn_dwconv_wgrad_planned(
        code, _lib.ptr(x), x.shape[0], _lib.ptr(g), _lib.ptr(plan.loc), _lib.ptr(plan.uptr),
        _lib.ptr(plan.urows), plan.umax, plan.total, rows, K, C, _lib.ptr(gw), _lib.ptr(ws), ws.numel(),
        _lib.stream()))
    if plan.overflow_rows is not None:
      gw += dw_wgrad(x, g.index_select(0, plan.overflow_rows), plan.overflow_table)
    return gw
  ws = _lib.workspace(L.ocnn_dwconv_wgrad_workspace_bytes(rows, K, C), x.device)
  _lib.check(L.ocnn_dwconv_wgrad(_lib.dtype_code(x), _lib.ptr(x), x.shape[0], _lib.ptr(g),
                                 _lib.ptr(table), rows, K, C, _lib.ptr(gw), _lib.ptr(ws),
                                 ws.numel(), _lib.stream()))
  return gw


class OctreeDWConvBase(OctreeConvBase):
  """Depth-wise engine (ocnn/nn/octree_dwconv.py:19-118)."""

  def __init__(self, in_channels: int, kernel_size: List[int] = [3], stride: int = 1,
               nempty: bool = False, max_buffer: int = int(2e8)):
    super().__init__(in_channels, in_channels, kernel_size, stride, nempty, max_buffer)
    self.weights_shape = (self.kdim, 1, self.out_channels)

  def is_conv_layer(self): return True

  def _dw_plan(self, data, inverse=False):
    """Tile plan of the table, when the staged depth-wise kernels take the shape."""
    code = _lib.DTYPE_CODE.get(data.dtype, -1)
    if not _lib.lib().ocnn_dwconv_gather_planned_supported(code, data.shape[0], self.kdim,
                                                           data.shape[1], 0):
      return None
    return self.octree._plan(self.neigh_depth, self.kernel, self.stride, self.nempty, inverse,
                             self.fine_h)

  def forward_gemm(self, data, weights, bias=None):
    return dw_gather(data, self.fine_h, self.neigh, weights, False, bias, self._dw_plan(data))

  def backward_gemm(self, grad, weights, bias=None):
    if self.symmetric:
      return dw_gather(grad, grad.shape[0], self.neigh, weights, True, bias, self._dw_plan(grad))
    return dw_gather(grad, grad.shape[0], self._inverse_table(), weights, False, bias,
                     self._dw_plan(grad, inverse=True))

  def weight_gemm(self, data, grad, out_transposed=False):
    return dw_wgrad(data, grad, self.neigh, self._dw_plan(data))


class OctreeDWConvFunction(Function):
  """Autograd wiring (ocnn/nn/octree_dwconv.py:121-155)."""

  @staticmethod
  def forward(ctx, data, weights, octree, depth: int, in_channels: int,
              kernel_size: List[int] = [3, 3, 3], stride: int = 1, nempty: bool = False,
              max_buffer: int = int(2e8)):
    eng = OctreeDWConvBase(in_channels, kernel_size, stride, nempty, max_buffer)
    eng.setup(octree, depth)
    eng.check_and_init(data)
    data = data.contiguous()
    weights = weights.to(data.dtype).contiguous()
    out = eng.forward_gemm(data, weights)
    ctx.save_for_backward(data, weights)
    ctx.eng = eng
    return out

  @staticmethod
  def backward(ctx, grad):
    data, weights = ctx.saved_tensors
    eng = ctx.eng
    grad = grad.contiguous()
    grad_out = eng.backward_gemm(grad, weights) if ctx.needs_input_grad[0] else None
    grad_w = eng.weight_gemm(data, grad) if ctx.needs_input_grad[1] else None
    return (grad_out, grad_w) + (None,) * 7


octree_dwconv = OctreeDWConvFunction.apply


class OctreeDWConv(OctreeDWConvBase, torch.nn.Module):
  """Depth-wise octree convolution (ocnn/nn/octree_dwconv.py:162-205):
  weights (kdim, 1, C); `bias` exists only when use_bias is set."""

  def __init__(self, in_channels: int, kernel_size: List[int] = [3], stride: int = 1,
               nempty: bool = False, use_bias: bool = False, max_buffer: int = int(2e8)):
    super().__init__(in_channels, kernel_size, stride, nempty, max_buffer)
    self.use_bias = use_bias
    self.weights = torch.nn.Parameter(torch.Tensor(*self.weights_shape))
    if self.use_bias:
      self.bias = torch.nn.Parameter(torch.Tensor(in_channels))
    self.reset_parameters()

  def reset_parameters(self):
    xavier_uniform_(self.weights)
    if self.use_bias:
      torch.nn.init.zeros_(self.bias)

  def forward(self, data: torch.Tensor, octree, depth: int):
    out = octree_dwconv(data, self.weights, octree, depth, self.in_channels, self.kernel_size,
                        self.stride, self.nempty, self.max_buffer)
    if self.use_bias:
      out = out + self.bias.to(out.dtype)
    if self.stride == 2 and not self.nempty:
      out = octree_pad(out, octree, depth - 1)
    return out

  def extra_repr(self) -> str:
    return ('in_channels={}, out_channels={}, kernel_size={}, stride={}, '
            'nempty={}, bias={}').format(self.in_channels, self.out_channels, self.kernel_size,
                                         self.stride, self.nempty, self.use_bias)
