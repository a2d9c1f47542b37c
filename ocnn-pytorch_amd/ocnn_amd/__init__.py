"""MI355X-native octree sparse-convolution hot path with the API of
octree-nn/ocnn-pytorch's ``ocnn`` package for that path (Octree, Points,
xyz2key/key2xyz, OctreeConv, OctreeDeconv, OctreeDWConv, octree_pad)."""

from . import octree, nn, utils, modules
from .octree import Octree, Points
from ._lib import lib as load_library

__version__ = '0.1.0'
__all__ = ['octree', 'nn', 'utils', 'modules', 'Octree', 'Points', 'load_library']
