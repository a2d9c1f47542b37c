"""Compositions of the hot-path layers with batch norm / ReLU / Linear under the class and
attribute names of ocnn/modules/modules.py and ocnn/modules/resblocks.py, so that networks
written against the reference (and their state_dicts) work unchanged.  The batch norm is a
BatchNorm1d subclass that runs on fused HIP kernels (statistics, normalise + ReLU in one pass)."""

from typing import List

import torch
import torch.nn
import torch.nn.functional as F

from .nn import OctreeConv, OctreeDeconv
from .nn.octree_conv import conv_gather, conv_wgrad, column_sum
from .nn.batchnorm import BatchNormRelu1d


class _LayerBn(torch.nn.Module):
  """layer -> BatchNorm1d [-> ReLU]; `name` is the attribute the layer is stored under."""

  def __init__(self, name, layer, channels, relu):
    super().__init__()
    self._name = name
    setattr(self, name, layer)
    self.bn = BatchNormRelu1d(channels, relu=relu)          # BatchNorm1d with the ReLU fused in
    if relu:
      self.relu = torch.nn.ReLU(inplace=True)               # (kept for the module tree; applied by bn)

  def forward(self, data, *args):
    return self.bn(getattr(self, self._name)(data, *args))


class OctreeConvBn(_LayerBn):
  """ocnn/modules/modules.py:32-51."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False):
    super().__init__('conv', OctreeConv(in_channels, out_channels, kernel_size, stride, nempty),
                     out_channels, False)


class OctreeConvBnRelu(_LayerBn):
  """ocnn/modules/modules.py:54-75."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False):
    super().__init__('conv', OctreeConv(in_channels, out_channels, kernel_size, stride, nempty),
                     out_channels, True)


class OctreeDeconvBnRelu(_LayerBn):
  """ocnn/modules/modules.py:78-99."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False):
    super().__init__('deconv', OctreeDeconv(in_channels, out_channels, kernel_size, stride, nempty),
                     out_channels, True)


_IDENTITY = {}


def _identity_table(rows, device):
  """(rows, 1) table [0, 1, ..]: row i reads row i."""
  key = (rows, str(device))
  if key not in _IDENTITY:
    if len(_IDENTITY) > 16:
      _IDENTITY.clear()
    _IDENTITY[key] = torch.arange(rows, dtype=torch.int32, device=device).view(rows, 1)
  return _IDENTITY[key]


class _RowsLinear(torch.autograd.Function):
  """y = x W^T + b on many rows through the one-slot form of the convolution kernels
  (weights (out, in) as torch.nn.Linear holds them)."""

  @staticmethod
  def forward(ctx, x, weight, bias):
    x = x.contiguous()
    w = weight.to(x.dtype).contiguous()
    ctx.save_for_backward(x, w)
    ctx.has_bias = bias is not None
    ctx.wdtype = weight.dtype
    rows = x.shape[0]
    return conv_gather(x, rows, _identity_table(rows, x.device), w.view(1, w.shape[0], w.shape[1]),
                       w.shape[0], True, False, None if bias is None else bias.to(x.dtype), None, dense=True)

  @staticmethod
  def backward(ctx, grad):
    x, w = ctx.saved_tensors
    grad = grad.contiguous()
    rows = x.shape[0]
    table = _identity_table(rows, x.device)
    gx = gw = gb = None
    if ctx.needs_input_grad[0]:
      gx = conv_gather(grad, rows, table, w.view(1, w.shape[0], w.shape[1]), w.shape[1], False, False,
                       None, None, dense=True)
    if ctx.needs_input_grad[1]:
      gw = conv_wgrad(x, grad, table, True, None, dense=True).view(w.shape).to(ctx.wdtype)
    if ctx.has_bias and ctx.needs_input_grad[2]:
      gb = column_sum(grad)
    return gx, gw, gb


class _RowsLinearNarrow(torch.autograd.Function):
  """y = x W^T + b for few output channels (a classification head: 64 -> 10 on a million
  rows).  Output and input gradient are the library's GEMMs; the weight gradient, a sum over
  all rows into a handful of numbers, is where the library's choice of kernel is slow (0.89 ms
  for 1.2 M x 64 x 10) and runs on this package's split reduction instead (fixed order)."""

  @staticmethod
  def forward(ctx, x, weight, bias):
    x = x.contiguous()
    ctx.save_for_backward(x, weight)
    ctx.has_bias = bias is not None
    return F.linear(x, weight.to(x.dtype), None if bias is None else bias.to(x.dtype))

  @staticmethod
  def backward(ctx, grad):
    x, weight = ctx.saved_tensors
    grad = grad.contiguous()
    rows = x.shape[0]
    gx = gw = gb = None
    if ctx.needs_input_grad[0]:
      gx = grad @ weight.to(grad.dtype)
    if ctx.needs_input_grad[1]:
      gw = conv_wgrad(x, grad, _identity_table(rows, x.device), True, None, dense=True)
      gw = gw.view(weight.shape).to(weight.dtype)
    if ctx.has_bias and ctx.needs_input_grad[2]:
      gb = column_sum(grad)
    return gx, gw, gb


class Conv1x1(torch.nn.Module):
  """ocnn/modules/modules.py:102-117: a 1x1x1 convolution on (N, C) rows is a Linear (same
  parameters as torch.nn.Linear; large 16-bit inputs run on this package's GEMM kernels)."""

  def __init__(self, in_channels: int, out_channels: int, use_bias: bool = False):
    super().__init__()
    self.linear = torch.nn.Linear(in_channels, out_channels, use_bias)

  def forward(self, data: torch.Tensor):
    lin = self.linear
    if (data.dim() == 2 and data.is_cuda and data.dtype in (torch.float16, torch.bfloat16) and
        data.shape[0] >= 4096 and lin.in_features % 32 == 0 and lin.out_features % 16 == 0):
      return _RowsLinear.apply(data, lin.weight, lin.bias)
    if (data.dim() == 2 and data.is_cuda and data.dtype in (torch.float16, torch.bfloat16) and
        data.shape[0] >= 65536 and lin.in_features % 32 == 0 and lin.out_features < 16):
      return _RowsLinearNarrow.apply(data, lin.weight, lin.bias)
    return lin(data)


class Conv1x1Bn(_LayerBn):
  """ocnn/modules/modules.py:120-134."""

  def __init__(self, in_channels: int, out_channels: int):
    super().__init__('conv', Conv1x1(in_channels, out_channels, use_bias=False), out_channels, False)


class Conv1x1BnRelu(_LayerBn):
  """ocnn/modules/modules.py:137-153."""

  def __init__(self, in_channels: int, out_channels: int):
    super().__init__('conv', Conv1x1(in_channels, out_channels, use_bias=False), out_channels, True)


class OctreeResBlock2(torch.nn.Module):
  """Two 3x3x3 convolutions with a (projected) shortcut, stride 1
  (ocnn/modules/resblocks.py:65-99)."""

  def __init__(self, in_channels, out_channels, stride=1, bottleneck=1, nempty=False):
    super().__init__()
    assert stride == 1, 'OctreeResBlock2: stride 1 only'
    self.in_channels, self.out_channels, self.stride = in_channels, out_channels, stride
    mid = int(out_channels / bottleneck)
    self.conv3x3a = OctreeConvBnRelu(in_channels, mid, nempty=nempty)
    self.conv3x3b = OctreeConvBn(mid, out_channels, nempty=nempty)
    if in_channels != out_channels:
      self.conv1x1 = Conv1x1Bn(in_channels, out_channels)
    self.relu = torch.nn.ReLU(inplace=True)

  def forward(self, data: torch.Tensor, octree, depth: int):
    out = self.conv3x3b.conv(self.conv3x3a(data, octree, depth), octree, depth)
    if self.in_channels != self.out_channels:
      data = self.conv1x1(data)
    # relu(bn(out) + data): the sum and the ReLU ride on the batch norm's pass over `out`
    return self.conv3x3b.bn(out, residual=data, relu=True)


class OctreeResBlocks(torch.nn.Module):
  """A chain of residual blocks (ocnn/modules/resblocks.py:134-159)."""

  def __init__(self, in_channels, out_channels, resblk_num, bottleneck=4, nempty=False,
               resblk=OctreeResBlock2, use_checkpoint=False):
    super().__init__()
    self.resblk_num = resblk_num
    self.use_checkpoint = use_checkpoint
    widths = [in_channels] + [out_channels] * resblk_num
    self.resblks = torch.nn.ModuleList(
        [resblk(widths[i], widths[i + 1], 1, bottleneck, nempty) for i in range(resblk_num)])

  def forward(self, data: torch.Tensor, octree, depth: int):
    for blk in self.resblks:
      if self.use_checkpoint:
        data = torch.utils.checkpoint.checkpoint(blk, data, octree, depth, use_reentrant=False)
      else:
        data = blk(data, octree, depth)
    return data


class InputFeature(torch.nn.Module):
  """The input signal stored in the octree (ocnn/modules/modules.py:288-305)."""

  def __init__(self, feature: str = 'NDF', nempty: bool = False):
    super().__init__()
    self.nempty = nempty
    self.feature = feature.upper()

  def forward(self, octree):
    return octree.get_input_feature(self.feature, self.nempty)

  def extra_repr(self) -> str:
    return 'feature={}, nempty={}'.format(self.feature, self.nempty)
