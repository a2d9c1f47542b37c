"""Morton ("shuffled") keys on the GPU; API of ocnn/octree/shuffled_key.py."""

from typing import Optional, Union

import torch

from .. import _lib


def xyz2key(x: torch.Tensor, y: torch.Tensor, z: torch.Tensor,
            b: Optional[Union[torch.Tensor, int]] = None, depth: int = 16):
  """Encodes coordinates (any dtype; truncated to int64 like ``.long()``) and
  an optional batch index (< 32768) into keys; depth < 17.
  Mirrors ocnn/octree/shuffled_key.py:60-90."""
  _lib.require_gpu(x, y, z)
  xs = [t.long().contiguous().view(-1) for t in (x, y, z)]
  n = xs[0].numel()
  bt = None
  if b is not None:
    if isinstance(b, torch.Tensor):
      bt = b.long().contiguous().view(-1)
    else:
      bt = torch.full((n,), int(b), dtype=torch.long, device=x.device)
  key = torch.empty(x.shape, dtype=torch.long, device=x.device)
  _lib.check(_lib.lib().ocnn_xyz2key(_lib.ptr(xs[0]), _lib.ptr(xs[1]), _lib.ptr(xs[2]),
                                     _lib.ptr(bt), n, depth, _lib.ptr(key), _lib.stream()))
  return key


def key2xyz(key: torch.Tensor, depth: int = 16):
  """Decodes keys into (x, y, z, b).  Mirrors ocnn/octree/shuffled_key.py:93-115."""
  _lib.require_gpu(key)
  k = key.long().contiguous()
  out = [torch.empty_like(k) for _ in range(4)]
  _lib.check(_lib.lib().ocnn_key2xyz(_lib.ptr(k), k.numel(), depth, _lib.ptr(out[0]),
                                     _lib.ptr(out[1]), _lib.ptr(out[2]), _lib.ptr(out[3]),
                                     _lib.stream()))
  return out[0], out[1], out[2], out[3]
