"""Table-level entry points with the signatures of the reference's implicit-GEMM
path (ocnn/nn/octree_conv_t.py, ocnn/nn/kernels/__init__.py): weights are
(Co, V, Ci), the table is (N, V) with -1 holes and must be centrally symmetric
(a 3x3x3 stride-1 table), as that path assumes."""

from typing import Optional, Tuple

import torch
from torch.autograd import Function

from .octree_conv import OctreeConv, column_sum, conv_gather, conv_wgrad


def _table32(neigh):
  return neigh if neigh.dtype == torch.int32 else neigh.int()


def conv_fwd_implicit_gemm_splitk(input, weight, bias, neighbor):
  """ocnn/nn/kernels/conv_fwd_implicit_gemm_splitk.py:118-150."""
  assert input.shape[1] == weight.shape[2], 'Incompatible dimensions'
  assert input.is_contiguous() and weight.is_contiguous() and neighbor.is_contiguous()
  w = weight.permute(1, 2, 0).contiguous()          # (V, Ci, Co)
  return conv_gather(input, input.shape[0], _table32(neighbor), w, weight.shape[0], False,
                     False, bias)


def conv_bwd_implicit_gemm_splitk(grad_output, input, weight, bias, neighbor, needs_input_grad
                                  ) -> Tuple[Optional[torch.Tensor], ...]:
  """ocnn/nn/kernels/conv_bwd_implicit_gemm_splitk.py:309-347."""
  assert grad_output.is_contiguous() and input.is_contiguous() and weight.is_contiguous()
  assert input.shape[1] == weight.shape[2], 'Incompatible dimensions'
  table = _table32(neighbor)
  gi = gw = gb = None
  if needs_input_grad[0]:
    w = weight.permute(1, 2, 0).contiguous()        # (V, Ci, Co) read transposed + mirrored
    gi = conv_gather(grad_output, grad_output.shape[0], table, w, weight.shape[2], True, True)
  if needs_input_grad[1]:
    gw = conv_wgrad(input, grad_output, table).permute(2, 0, 1).contiguous()   # (Co, V, Ci)
  if len(needs_input_grad) > 2 and needs_input_grad[2]:
    gb = column_sum(grad_output)
  return gi, gw, gb


class OctreeConvTritonFunction(Function):
  """ocnn/nn/octree_conv_t.py:27-52."""

  @staticmethod
  def forward(ctx, data, weights, bias, neigh):
    data = data.contiguous()
    weights = weights.contiguous().to(data.dtype)
    neigh = neigh.contiguous()
    if bias is not None:
      bias = bias.contiguous().to(data.dtype)
    out = conv_fwd_implicit_gemm_splitk(data, weights, bias, neigh)
    ctx.save_for_backward(data, weights, bias, neigh)
    return out

  @staticmethod
  def backward(ctx, grad):
    data, weights, bias, neigh = ctx.saved_tensors
    gi, gw, gb = conv_bwd_implicit_gemm_splitk(grad.contiguous(), data, weights, bias, neigh,
                                               ctx.needs_input_grad)
    return gi, gw, gb, None


octree_conv_triton = OctreeConvTritonFunction.apply


class OctreeConvTriton(OctreeConv):
  """Name kept for drop-in use (ocnn/nn/octree_conv_t.py:59-130): 3x3x3,
  stride 1 only, like the class it stands in for."""

  def __init__(self, in_channels, out_channels, kernel_size=[3], stride=1, nempty=False,
               method='triton', use_bias=False, max_buffer=int(2e8)):
    super().__init__(in_channels, out_channels, kernel_size, stride, nempty, method, use_bias,
                     max_buffer)
    assert self.stride == 1, 'Only stride=1 is supported now.'
    assert self.kernel == '333', 'Only kernel_size=[3,3,3] is supported now.'


OctreeConvT = OctreeConvTriton


def convert_conv_triton(module: torch.nn.Module) -> torch.nn.Module:
  """Every OctreeConv already runs on the HIP engine, so there is nothing to
  convert (ocnn/nn/octree_conv_t.py:137-160)."""
  return module
