"""The segmentation U-Net of the reference (ocnn/models/unet.py:16-105) assembled from this
package's layers: same constructor, same sub-module names (`conv1`, `downsample`, `encoder`,
`upsample`, `decoder`, `octree_interp`, `header`), so its state_dicts load unchanged.

Four levels down, four levels up.  Level i of the encoder halves the resolution with a 2x2x2
stride-2 convolution and runs `ENCODER_BLOCKS[i]` residual blocks; level i of the decoder
doubles it with a 2x2x2 stride-2 deconvolution, concatenates the encoder's features of that
depth in front and runs `DECODER_BLOCKS[i]` residual blocks.  The features of the finest
level are interpolated at the query points and classified by a 1x1 head."""

import torch
import torch.nn

from . import modules
from .nn import OctreeInterp

ENCODER_CHANNELS = (32, 32, 64, 128, 256)
DECODER_CHANNELS = (256, 256, 128, 96, 96)
ENCODER_BLOCKS = (2, 3, 4, 6)
DECODER_BLOCKS = (2, 2, 2, 2)
HEAD_CHANNELS = 64


class UNet(torch.nn.Module):

  def __init__(self, in_channels: int, out_channels: int, interp: str = 'linear',
               nempty: bool = False, **kwargs):
    super().__init__()
    self.in_channels, self.out_channels, self.nempty = in_channels, out_channels, nempty
    enc, dec = ENCODER_CHANNELS, DECODER_CHANNELS
    self.encoder_stages, self.decoder_stages = len(ENCODER_BLOCKS), len(DECODER_BLOCKS)
    levels = range(self.encoder_stages)
    self.conv1 = modules.OctreeConvBnRelu(in_channels, enc[0], nempty=nempty)
    self.downsample = torch.nn.ModuleList(
        modules.OctreeConvBnRelu(enc[i], enc[i + 1], [2], 2, nempty) for i in levels)
    self.encoder = torch.nn.ModuleList(
        modules.OctreeResBlocks(enc[i + 1], enc[i + 1], ENCODER_BLOCKS[i], 1, nempty) for i in levels)
    levels = range(self.decoder_stages)
    self.upsample = torch.nn.ModuleList(
        modules.OctreeDeconvBnRelu(dec[i], dec[i + 1], [2], 2, nempty) for i in levels)
    # skip connection: the encoder's features of the same depth come first
    self.decoder = torch.nn.ModuleList(
        modules.OctreeResBlocks(dec[i + 1] + enc[-i - 2], dec[i + 1], DECODER_BLOCKS[i], 1, nempty)
        for i in levels)
    self.octree_interp = OctreeInterp(interp, nempty)
    self.header = torch.nn.Sequential(modules.Conv1x1BnRelu(dec[-1], HEAD_CHANNELS),
                                      modules.Conv1x1(HEAD_CHANNELS, out_channels, use_bias=True))

  def unet_encoder(self, data, octree, depth: int):
    """{depth: features} for depth .. depth - 4."""
    feats = {depth: self.conv1(data, octree, depth)}
    for i, (down, blocks) in enumerate(zip(self.downsample, self.encoder)):
      feats[depth - i - 1] = blocks(down(feats[depth - i], octree, depth - i), octree, depth - i - 1)
    return feats

  def unet_decoder(self, feats, octree, depth: int):
    """From the coarsest features at `depth` up to depth + 4."""
    x = feats[depth]
    for i, (up, blocks) in enumerate(zip(self.upsample, self.decoder)):
      x = torch.cat([feats[depth + i + 1], up(x, octree, depth + i)], dim=1)
      x = blocks(x, octree, depth + i + 1)
    return x

  def forward(self, data: torch.Tensor, octree, depth: int, query_pts: torch.Tensor):
    """query_pts (N, 4): xyz in [-1, 1] and the batch index (rescaled in place to octree
    coordinates, as the reference's OctreeInterp does).  Returns (N, out_channels) logits."""
    feats = self.unet_encoder(data, octree, depth)
    coarse = depth - self.encoder_stages
    x = self.unet_decoder(feats, octree, coarse)
    return self.header(self.octree_interp(x, octree, coarse + self.decoder_stages, query_pts))
