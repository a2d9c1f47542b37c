"""Group convolution with the API of ocnn/nn/octree_gconv.py: one OctreeConv per group over
its slice of the channels (the reference does the same; `convs` holds the per-group layers,
so its state_dicts load)."""

from typing import List

import torch
import torch.nn

from .octree_conv import OctreeConv


class OctreeGroupConv(torch.nn.Module):
  """ocnn/nn/octree_gconv.py:16-79."""

  def __init__(self, in_channels: int, out_channels: int, kernel_size: List[int] = [3],
               stride: int = 1, nempty: bool = False, use_bias: bool = False, group: int = 1):
    super().__init__()
    assert in_channels % group == 0 and out_channels % group == 0
    self.group = group
    self.in_channels = in_channels
    self.out_channels = out_channels
    self.in_channels_per_group = in_channels // group
    self.out_channels_per_group = out_channels // group
    self.convs = torch.nn.ModuleList(
        [OctreeConv(self.in_channels_per_group, self.out_channels_per_group, kernel_size, stride,
                    nempty, use_bias=use_bias) for _ in range(group)])

  def forward(self, data: torch.Tensor, octree, depth: int):
    assert data.shape[1] == self.in_channels
    parts = torch.split(data, self.in_channels_per_group, dim=1)
    return torch.cat([conv(part.contiguous(), octree, depth) for conv, part in zip(self.convs, parts)], dim=1)

  def extra_repr(self) -> str:
    return 'in_channels={}, out_channels={}, group={}'.format(self.in_channels, self.out_channels, self.group)
