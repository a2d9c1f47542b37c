"""Point-cloud container with the part of ocnn/octree/points.py the octree
build needs: construction checks, normalize, merge, device moves."""

from typing import List, Optional, Union

import torch


class Points:
  """points (N,3) with optional normals (N,3), features (N,C), labels (N,K),
  batch_id (N,1).  Mirrors ocnn/octree/points.py:14-70."""

  def __init__(self, points: torch.Tensor, normals: Optional[torch.Tensor] = None,
               features: Optional[torch.Tensor] = None, labels: Optional[torch.Tensor] = None,
               batch_id: Optional[torch.Tensor] = None, batch_size: int = 1):
    self.points = points
    self.normals = normals
    self.features = features
    self.labels = labels
    self.batch_id = batch_id
    self.batch_size = batch_size
    self.device = points.device
    self.batch_npt = None
    self.check_input()

  def check_input(self):
    n = self.points.size(0)
    assert self.points.dim() == 2 and self.points.size(1) == 3
    if self.normals is not None:
      assert self.normals.dim() == 2 and self.normals.size(1) == 3 and self.normals.size(0) == n
    if self.features is not None:
      assert self.features.dim() == 2 and self.features.size(0) == n
    if self.labels is not None:
      assert self.labels.dim() in (1, 2) and self.labels.size(0) == n
      if self.labels.dim() == 1:
        self.labels = self.labels.unsqueeze(1)
    if self.batch_id is not None:
      assert self.batch_id.dim() in (1, 2) and self.batch_id.size(0) == n
      if self.batch_id.dim() == 1:
        self.batch_id = self.batch_id.unsqueeze(1)
      assert self.batch_id.size(1) == 1
      assert self.batch_size == self.batch_id.max().item() + 1

  @property
  def npt(self):
    return self.points.shape[0]

  def bbox(self):
    return self.points.min(dim=0)[0], self.points.max(dim=0)[0]

  def normalize(self, bbmin, bbmax, scale: float, inplace: bool = False):
    """Maps [bbmin, bbmax] to [0, scale] (ocnn/octree/points.py:223-244)."""
    box_size = bbmax - bbmin
    if type(box_size) is torch.Tensor:
      box_size = box_size.max().item()
    assert box_size > 0, 'The bounding box size must be greater than 0.'
    points = (self.points - bbmin) * (scale / box_size)
    if inplace:
      self.points = points
    return points

  def to(self, device: Union[torch.device, str], non_blocking: bool = False):
    if isinstance(device, str):
      device = torch.device(device)
    if self.device == device:
      return self

    def mv(t):
      return None if t is None else t.to(device, non_blocking=non_blocking)

    out = Points(mv(self.points), mv(self.normals), mv(self.features), mv(self.labels),
                 mv(self.batch_id), self.batch_size)
    out.batch_npt = self.batch_npt
    return out

  def cuda(self, non_blocking: bool = False):
    return self.to('cuda', non_blocking)

  def cpu(self):
    return self.to('cpu')

  def merge_points(self, points: List['Points'], update_batch_info: bool = True):
    """Concatenates clouds into one batch (ocnn/octree/points.py:331-357);
    batch ids are stored in the points' float dtype, as the reference does."""
    def cat(name):
      return torch.cat([getattr(p, name) for p in points], dim=0)

    self.points = cat('points')
    for name in ('normals', 'features', 'labels'):
      if getattr(points[0], name) is not None:
        setattr(self, name, cat(name))
    self.device = points[0].device
    if update_batch_info:
      self.batch_size = len(points)
      self.batch_npt = torch.tensor([p.npt for p in points], dtype=torch.long)
      self.batch_id = torch.cat([p.points.new_full((p.npt, 1), i)
                                 for i, p in enumerate(points)], dim=0)
    return self

  @classmethod
  def init_points(cls, device=None, batch_size: int = 1):
    pts = torch.zeros(batch_size, 3, device=device)
    bid = torch.arange(batch_size, device=device).unsqueeze(1) if batch_size > 1 else None
    return cls(pts, batch_size=batch_size, batch_id=bid)


def merge_points(points: List['Points'], update_batch_info: bool = True):
  assert len(points) > 0, 'The input points list is empty.'
  out = Points.init_points(points[0].device, batch_size=len(points))
  return out.merge_points(points, update_batch_info)
