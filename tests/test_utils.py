"""The helpers of ocnn/utils.py that the hot path leans on, with the reference's own test
vectors (test/test_utils.py:17-46) and the closed forms of the rest.  CPU only."""

import torch

from ocnn_amd import utils


def test_scatter_add_reference_vector():
  src = torch.arange(1, 11).view(2, 5)
  idx = torch.tensor([0, 1, 3, 2, 0])
  want = torch.tensor([[6, 2, 4, 3, 0], [16, 7, 9, 8, 0]])
  assert torch.equal(utils.scatter_add(src, idx, dim=1, dim_size=5), want)
  # rows scattered along dim 0 (how the octree build averages the points of a leaf), size
  # taken from the largest index, accumulation into a given tensor
  rows = torch.tensor([[1., 2.], [3., 4.], [5., 6.]])
  assert torch.equal(utils.scatter_add(rows, torch.tensor([2, 0, 2]), dim=0),
                     torch.tensor([[3., 4.], [0., 0.], [6., 8.]]))
  out = torch.ones(3, 2)
  res = utils.scatter_add(rows, torch.tensor([1, 1, 1]), dim=0, out=out)
  assert res is out and torch.equal(out, torch.tensor([[1., 1.], [10., 13.], [1., 1.]]))
  assert utils.scatter_add(torch.zeros(0, 2), torch.zeros(0, dtype=torch.long), dim=0).shape == (0, 2)


def test_cumsum_reference_vectors():
  data = torch.tensor([[1, 2, 3], [4, 5, 6]])
  assert torch.equal(utils.cumsum(data, dim=1, exclusive=False), torch.tensor([[1, 3, 6], [4, 9, 15]]))
  assert torch.equal(utils.cumsum(data, dim=1, exclusive=True), torch.tensor([[0, 1, 3, 6], [0, 4, 9, 15]]))
  assert torch.equal(utils.cumsum(data, dim=0, exclusive=True), torch.tensor([[0, 0, 0], [1, 2, 3], [5, 7, 9]]))


def test_resize_with_last_val_returns_copy():
  data = [2]
  out = utils.resize_with_last_val(data)
  assert out == [2, 2, 2] and data == [2] and out is not data
  assert utils.resize_with_last_val([3, 1]) == [3, 1, 1]
  assert utils.list2str([3, 1, 1]) == '311'


def test_range_grid_order():
  g = utils.range_grid(-1, 1)
  assert g.shape == (27, 3) and g.dtype == torch.long
  # slot k = (dx + 1) * 9 + (dy + 1) * 3 + (dz + 1): x slowest
  for k in range(27):
    assert g[k].tolist() == [k // 9 - 1, (k // 3) % 3 - 1, k % 3 - 1]
  assert utils.range_grid(0, 1).tolist() == [[x, y, z] for x in (0, 1) for y in (0, 1) for z in (0, 1)]


def test_trunc_div_rounds_toward_zero():
  a = torch.tensor([-5, -4, -1, 0, 1, 4, 5])
  assert utils.trunc_div(a, 2).tolist() == [-2, -2, 0, 0, 0, 2, 2]
  assert utils.trunc_div(a, 2).dtype == torch.long


def test_xavier_uniform_bound():
  w = torch.empty(27, 8, 16)
  torch.manual_seed(0)
  utils.xavier_uniform_(w)
  bound = (3.0 ** 0.5) * (2.0 / (27 * 8 + 27 * 16)) ** 0.5
  assert float(w.abs().max()) <= bound and float(w.abs().max()) > 0.9 * bound
  assert abs(float(w.mean())) < 0.05 * bound
