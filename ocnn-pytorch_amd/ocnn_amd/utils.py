"""Small helpers with the semantics of the reference's ocnn/utils.py."""

import math
from typing import Optional

import torch

__all__ = ['trunc_div', 'meshgrid', 'range_grid', 'cumsum', 'scatter_add', 'xavier_uniform_',
           'resize_with_last_val', 'list2str']


def trunc_div(input, other):
  """C-style integer division (ocnn/utils.py:21-31)."""
  return torch.div(input, other, rounding_mode='trunc')


def meshgrid(*tensors, indexing: Optional[str] = None):
  return torch.meshgrid(*tensors, indexing=indexing)


def range_grid(min: int, max: int, device='cpu'):
  """All integer points of [min, max]^3, x slowest (ocnn/utils.py:46-74)."""
  r = torch.arange(min, max + 1, dtype=torch.long, device=device)
  n = r.numel()
  x = r.view(n, 1, 1).expand(n, n, n)
  y = r.view(1, n, 1).expand(n, n, n)
  z = r.view(1, 1, n).expand(n, n, n)
  return torch.stack([x, y, z], dim=-1).reshape(-1, 3)


def cumsum(data: torch.Tensor, dim: int, exclusive: bool = False):
  """torch.cumsum; exclusive=True prepends a zero, growing `dim` by one
  (ocnn/utils.py:77-96)."""
  out = torch.cumsum(data, dim)
  if exclusive:
    shape = list(data.shape)
    shape[dim] = 1
    out = torch.cat([out.new_zeros(shape), out], dim)
  return out


def scatter_add(src: torch.Tensor, index: torch.Tensor, dim: int = -1,
                out: Optional[torch.Tensor] = None, dim_size: Optional[int] = None):
  """Row-broadcast scatter_add_ (ocnn/utils.py:117-147)."""
  if dim < 0:
    dim = src.dim() + dim
  if index.dim() == 1:
    shape = [1] * src.dim()
    shape[dim] = index.numel()
    index = index.view(shape)
  while index.dim() < src.dim():
    index = index.unsqueeze(-1)
  index = index.expand_as(src)
  if out is None:
    size = list(src.shape)
    if dim_size is not None:
      size[dim] = dim_size
    elif index.numel() == 0:
      size[dim] = 0
    else:
      size[dim] = int(index.max()) + 1
    out = torch.zeros(size, dtype=src.dtype, device=src.device)
  return out.scatter_add_(dim, index, src)


def xavier_uniform_(weights: torch.Tensor):
  """Xavier-uniform for (kdim, in, out) weights: fan_in = kdim*in, fan_out =
  kdim*out (ocnn/utils.py:150-166)."""
  kdim, cin, cout = weights.shape
  bound = math.sqrt(3.0) * math.sqrt(2.0 / float(kdim * cin + kdim * cout))
  torch.nn.init.uniform_(weights, -bound, bound)


def resize_with_last_val(list_in: list, num: int = 3):
  assert type(list_in) is list and len(list_in) < num + 1
  return list(list_in) + [list_in[-1]] * (num - len(list_in))


def list2str(list_in: list):
  return ''.join(str(x) for x in list_in)
