"""Seeded synthetic point clouds for benchmarks and tests (CPU float32 tensors).

Every cloud lies strictly inside [-1, 1]^3 and carries analytic unit normals.
"""

import math

import torch


def _gen(seed):
  g = torch.Generator()
  g.manual_seed(int(seed))
  return g


def sphere_points(n, g, radius=0.99, center=(0.0, 0.0, 0.0)):
  d = torch.randn(n, 3, generator=g)
  d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-12)
  return d * radius + torch.tensor(center, dtype=torch.float32), d


def box_points(n, g, lo, hi):
  """Uniform on the surface of the axis-aligned box [lo, hi] (area weighted)."""
  lo = torch.tensor(lo, dtype=torch.float32)
  hi = torch.tensor(hi, dtype=torch.float32)
  ext = hi - lo
  area = torch.stack([ext[1] * ext[2], ext[0] * ext[2], ext[0] * ext[1]]).repeat_interleave(2)
  face = torch.multinomial(area / area.sum(), n, replacement=True, generator=g)
  axis, side = face // 2, face % 2
  p = lo + torch.rand(n, 3, generator=g) * ext
  rows = torch.arange(n)
  p[rows, axis] = torch.where(side == 1, hi[axis], lo[axis])
  nrm = torch.zeros(n, 3)
  nrm[rows, axis] = side.float() * 2 - 1
  return p, nrm


def plane_points(n, g, normal, offset, half=0.98):
  """Points of the plane {x : <x, normal> = offset} inside the cube (rejection)."""
  nvec = torch.tensor(normal, dtype=torch.float32)
  nvec = nvec / nvec.norm()
  out = []
  got = 0
  while got < n:
    q = (torch.rand(2 * n, 3, generator=g) * 2 - 1) * half
    q = q - ((q @ nvec) - offset).unsqueeze(1) * nvec
    q = q[(q.abs() <= half).all(1)]
    out.append(q)
    got += q.shape[0]
  p = torch.cat(out)[:n]
  return p, nvec.expand(n, 3).clone()


def sphere_cloud(n=20000, seed=1000):
  """Config 0: points on the unit sphere scaled by 0.99, normals = direction."""
  return sphere_points(n, _gen(seed))


def mixed_cloud(n=100000, seed=1001, n_spheres=3, n_boxes=2):
  """Configs 1/2: spheres (radius U[0.1,0.5]) and axis-aligned boxes, each
  fully inside 0.98 * [-1,1]^3, equal share of the points."""
  g = _gen(seed)
  parts = n_spheres + n_boxes
  per = [n // parts + (1 if i < n % parts else 0) for i in range(parts)]
  pts, nrm = [], []
  for i in range(n_spheres):
    r = 0.1 + 0.4 * torch.rand(1, generator=g).item()
    c = ((torch.rand(3, generator=g) * 2 - 1) * (0.98 - r)).tolist()
    p, m = sphere_points(per[i], g, r, c)
    pts.append(p)
    nrm.append(m)
  for i in range(n_boxes):
    a = (torch.rand(3, generator=g) * 2 - 1) * 0.98
    b = (torch.rand(3, generator=g) * 2 - 1) * 0.98
    lo, hi = torch.minimum(a, b), torch.maximum(a, b)
    hi = torch.maximum(hi, lo + 0.05).clamp(max=0.98)
    p, m = box_points(per[n_spheres + i], g, lo.tolist(), hi.tolist())
    pts.append(p)
    nrm.append(m)
  return torch.cat(pts), torch.cat(nrm)


def planes_cloud(n=250000, seed=1003, n_planes=4, n_spheres=3):
  """Config 3: random planes clipped to the cube plus spheres."""
  g = _gen(seed)
  parts = n_planes + n_spheres
  per = [n // parts + (1 if i < n % parts else 0) for i in range(parts)]
  pts, nrm = [], []
  for i in range(n_planes):
    normal = torch.randn(3, generator=g).tolist()
    offset = (torch.rand(1, generator=g).item() * 2 - 1) * 0.5
    p, m = plane_points(per[i], g, normal, offset)
    pts.append(p)
    nrm.append(m)
  for i in range(n_spheres):
    r = 0.1 + 0.4 * torch.rand(1, generator=g).item()
    c = ((torch.rand(3, generator=g) * 2 - 1) * (0.98 - r)).tolist()
    p, m = sphere_points(per[n_planes + i], g, r, c)
    pts.append(p)
    nrm.append(m)
  return torch.cat(pts), torch.cat(nrm)


def rect_points(n, g, axis, level, lo, hi, sign):
  """Uniform on the axis-aligned rectangle {x[axis] = level, lo <= x <= hi on the other two axes};
  normal = sign along the axis."""
  lo = torch.tensor(lo, dtype=torch.float32)
  hi = torch.tensor(hi, dtype=torch.float32)
  p = lo + torch.rand(n, 3, generator=g) * (hi - lo)
  p[:, axis] = level
  nrm = torch.zeros(n, 3)
  nrm[:, axis] = float(sign)
  return p, nrm


def indoor_cloud(n=150000, seed=1004, min_boxes=10, max_boxes=20):
  """Config 4: an indoor-like scene: the floor of a room, two to four of its walls, and 10 - 20
  random axis-aligned boxes standing on the floor (furniture).  Points are spread over the
  surfaces in proportion to their areas; normals point into the room (floor, walls) or out of
  the boxes."""
  g = _gen(seed)
  u = lambda: torch.rand(1, generator=g).item()
  half, floor = 0.95, -0.9
  top = floor + 0.9 + 0.8 * u()                           # height of the walls
  parts = [('rect', (2, floor, (-half, -half, floor), (half, half, floor), 1.0), (2 * half) ** 2)]
  walls = [(0, -half, 1.0), (0, half, -1.0), (1, -half, 1.0), (1, half, -1.0)]
  order = torch.randperm(4, generator=g).tolist()
  for w in order[:2 + int(u() * 3) % 3]:
    axis, level, sign = walls[w]
    lo = [-half, -half, floor]
    hi = [half, half, top]
    lo[axis] = hi[axis] = level
    parts.append(('rect', (axis, level, tuple(lo), tuple(hi), sign), 2 * half * (top - floor)))
  n_boxes = min_boxes + int(u() * (max_boxes - min_boxes + 1)) % (max_boxes - min_boxes + 1)
  for _ in range(n_boxes):
    ext = [0.08 + 0.4 * u(), 0.08 + 0.4 * u(), 0.08 + 0.6 * u()]
    cx = (u() * 2 - 1) * (half - 0.02 - ext[0] / 2)
    cy = (u() * 2 - 1) * (half - 0.02 - ext[1] / 2)
    lo = (cx - ext[0] / 2, cy - ext[1] / 2, floor)
    hi = (cx + ext[0] / 2, cy + ext[1] / 2, min(floor + ext[2], 0.97))
    e = [h - l for l, h in zip(lo, hi)]
    parts.append(('box', (lo, hi), 2 * (e[0] * e[1] + e[1] * e[2] + e[0] * e[2])))
  area = torch.tensor([a for _, _, a in parts])
  which = torch.multinomial(area / area.sum(), n, replacement=True, generator=g)
  counts = torch.bincount(which, minlength=len(parts)).tolist()
  pts, nrm = [], []
  for (kind, args, _), c in zip(parts, counts):
    if c == 0:
      continue
    p, m = rect_points(c, g, *args) if kind == 'rect' else box_points(c, g, *args)
    pts.append(p)
    nrm.append(m)
  return torch.cat(pts), torch.cat(nrm)


def shell_voxels(depth, device='cpu', thickness=1.25):
  """Integer coordinates of the cells of the 2^depth grid whose centre lies within `thickness` cells
  inside the sphere inscribed in the grid: the octree of the reference's layer benchmark
  (test/utils.py:43-70; 3 840 / 15 192 / 64 160 / 252 392 / 1 026 536 / 4 113 056 cells at depths
  5 .. 10, test/benchmark_conv.py:23-31).  Deterministic; x-major order."""
  res = 1 << depth
  half = res / 2.0
  axis = torch.arange(res, device=device, dtype=torch.float32) - half + 0.5
  yz2 = (axis * axis).view(-1, 1) + (axis * axis).view(1, -1)                # (res, res)
  lo2 = max(half - thickness, 0.0)
  cells = []
  for x0 in range(0, res, 32):                                                # slabs of 32 planes
    d = (yz2.unsqueeze(0) + (axis[x0:x0 + 32] ** 2).view(-1, 1, 1)).sqrt()
    at = torch.nonzero((d <= half) & (d >= lo2))
    at[:, 0] += x0
    cells.append(at)
  return torch.cat(cells).int()


def shell_points(depth, device='cpu'):
  """The cells of shell_voxels as points in [-1, 1)^3 (each at its cell's lower corner, so that an
  octree of the same depth has exactly these cells as leaves)."""
  return shell_voxels(depth, device).float() / float(1 << depth) * 2.0 - 1.0


def batch_clouds(maker, batch, seed, **kw):
  """`batch` clouds -> (points, normals, batch_id as float32 (N,1))."""
  pts, nrm, bid = [], [], []
  for b in range(batch):
    p, m = maker(seed=seed * 100 + b, **kw)
    pts.append(p)
    nrm.append(m)
    bid.append(torch.full((p.shape[0], 1), float(b)))
  return torch.cat(pts), torch.cat(nrm), torch.cat(bid)
