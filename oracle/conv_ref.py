"""CPU restatement of the reference's octree convolution engine.

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this file.

Two forms of the same algorithm live here:

* the *literal definition* in numpy (any float dtype, normally fp64), one slot
  of the kernel at a time, used as the value oracle;
* ``BlockGemmCPU``: the chunked gather -> mm -> scatter_add form the reference
  runs on a CPU (ocnn/nn/octree_conv.py:115-202) written with torch CPU ops,
  used as the timed CPU baseline and cross-checked against the definition.

Shapes follow ocnn/nn/octree_conv.py:26-100: ``W`` is (K, in_conv, out_conv);
``table`` is the (rows, K) neighbour table from ``get_neigh`` with -1 holes.
"""

import numpy as np

from .octree_ref import LUT_KERNEL  # noqa: F401  (re-exported for tests)


# --------------------------------------------------------------------------
# engine: literal definitions
# --------------------------------------------------------------------------

def forward_gemm(data, W, table):
  """octree_conv.py:115-143: out[i] = sum_k [t_ik >= 0] data[t_ik] @ W[k]."""
  R, K = table.shape
  out = np.zeros((R, W.shape[2]), data.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    out[v] += data[t[v]] @ W[k]
  return out


def backward_gemm(grad, W, table, rows_in):
  """octree_conv.py:145-168: gin[t_ik] += grad[i] @ W[k]^T for valid (i, k)."""
  R, K = table.shape
  out = np.zeros((rows_in, W.shape[1]), grad.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    np.add.at(out, t[v], grad[v] @ W[k].T)
  return out


def weight_gemm(data, grad, table):
  """octree_conv.py:170-202: gW[k] = sum_i [t_ik >= 0] data[t_ik]^T (x) grad[i]."""
  R, K = table.shape
  out = np.zeros((K, data.shape[1], grad.shape[1]), data.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    out[k] = data[t[v]].T @ grad[v]
  return out


def dw_forward(data, W, table):
  """octree_dwconv.py:30-58: out[i,c] = sum_k data[t_ik,c] * w[k,c]."""
  R, K = table.shape
  w = W.reshape(K, -1)
  out = np.zeros((R, data.shape[1]), data.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    out[v] += data[t[v]] * w[k]
  return out


def dw_backward(grad, W, table, rows_in):
  """octree_dwconv.py:60-85: gin[t_ik,c] += grad[i,c] * w[k,c]."""
  R, K = table.shape
  w = W.reshape(K, -1)
  out = np.zeros((rows_in, grad.shape[1]), grad.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    np.add.at(out, t[v], grad[v] * w[k])
  return out


def dw_weight(data, grad, table):
  """octree_dwconv.py:87-118: gw[k,c] = sum_i data[t_ik,c] * grad[i,c]."""
  R, K = table.shape
  out = np.zeros((K, 1, data.shape[1]), data.dtype)
  for k in range(K):
    t = table[:, k]
    v = t >= 0
    out[k, 0] = (data[t[v]] * grad[v]).sum(0)
  return out


def octree_pad(data, oct, depth, val=0.0):
  """ocnn/nn/octree_pad.py:13-29."""
  out = np.full((int(oct.nnum[depth]), data.shape[1]), val, data.dtype)
  out[oct.nempty_index(depth)] = data
  return out


def octree_depad(data, oct, depth):
  """ocnn/nn/octree_pad.py:32-39."""
  return data[oct.nempty_index(depth)]


def octree2col(data, table):
  """ocnn/nn/octree2col.py:15-38 on a given table: (rows, K, C), zeros at -1 entries."""
  out = np.zeros((table.shape[0], table.shape[1], data.shape[1]), data.dtype)
  valid = table >= 0
  out[valid] = data[table[valid]]
  return out


def col2octree(col, table, rows_in):
  """ocnn/nn/octree2col.py:41-53: out[t_ik] += col[i, k] over the valid entries."""
  out = np.zeros((rows_in, col.shape[2]), col.dtype)
  valid = table >= 0
  np.add.at(out, table[valid], col[valid])
  return out


# --------------------------------------------------------------------------
# layer level: shapes as in OctreeConvBase.setup (octree_conv.py:51-100)
# --------------------------------------------------------------------------

def kernel_str(kernel_size):
  ks = list(kernel_size)
  while len(ks) < 3:
    ks.append(ks[-1])
  return ''.join(str(k) for k in ks)


class LayerShapes:
  """in/out heights and the neighbour table of one layer call."""

  def __init__(self, oct, depth, kernel_size, stride, nempty, is_conv):
    self.kernel = kernel_str(kernel_size)
    in_depth = out_depth = neigh_depth = depth
    if stride == 2:
      if is_conv:
        out_depth = depth - 1
      else:
        out_depth = depth + 1
        neigh_depth = depth + 1
    if nempty:
      in_h, out_h = oct.nnum_nempty[in_depth], oct.nnum_nempty[out_depth]
    else:
      in_h, out_h = oct.nnum[in_depth], oct.nnum[out_depth]
      if stride == 2:
        if is_conv:
          out_h = oct.nnum_nempty[out_depth]
        else:
          in_h = oct.nnum_nempty[in_depth]
    self.in_h, self.out_h = int(in_h), int(out_h)
    self.table = oct.get_neigh(neigh_depth, self.kernel, stride, nempty)


def conv_layer(oct, data, W, depth, kernel_size=(3,), stride=1, nempty=False,
               bias=None, grad=None):
  """OctreeConv.forward (octree_conv.py:401-421) and, when ``grad`` (the
  gradient w.r.t. the returned tensor) is given, its backward
  (octree_conv.py:239-254).  Returns out or (out, gdata, gW, gbias)."""
  s = LayerShapes(oct, depth, kernel_size, stride, nempty, True)
  assert data.shape[0] == s.in_h, 'The shape of input data is wrong'
  out = forward_gemm(data, W, s.table)
  assert out.shape[0] == s.out_h
  if bias is not None:
    out = out + bias
  padded = stride == 2 and not nempty
  res = octree_pad(out, oct, depth - 1) if padded else out
  if grad is None:
    return res
  g = octree_depad(grad, oct, depth - 1) if padded else grad
  gdata = backward_gemm(g, W, s.table, s.in_h)
  gW = weight_gemm(data, g, s.table)
  return res, gdata, gW, g.sum(0)


def deconv_layer(oct, data, W, depth, kernel_size=(3,), stride=1, nempty=False,
                 bias=None, grad=None):
  """OctreeDeconv.forward (octree_conv.py:441-466) / backward (:277-292).
  ``W`` is (K, out_channels, in_channels)."""
  s = LayerShapes(oct, depth, kernel_size, stride, nempty, False)
  depad = stride == 2 and not nempty
  x = octree_depad(data, oct, depth) if depad else data
  assert x.shape[0] == s.in_h, 'The shape of input data is wrong'
  out = backward_gemm(x, W, s.table, s.out_h)
  if bias is not None:
    out = out + bias
  if grad is None:
    return out
  gx = forward_gemm(grad, W, s.table)
  gW = weight_gemm(grad, x, s.table)
  if depad:
    full = np.zeros_like(data)
    full[oct.nempty_index(depth)] = gx
    gx = full
  return out, gx, gW, grad.sum(0)


def dwconv_layer(oct, data, W, depth, kernel_size=(3,), stride=1, nempty=False,
                 bias=None, grad=None):
  """OctreeDWConv.forward (octree_dwconv.py:188-200) / backward (:140-155)."""
  s = LayerShapes(oct, depth, kernel_size, stride, nempty, True)
  assert data.shape[0] == s.in_h, 'The shape of input data is wrong'
  out = dw_forward(data, W, s.table)
  if bias is not None:
    out = out + bias
  padded = stride == 2 and not nempty
  res = octree_pad(out, oct, depth - 1) if padded else out
  if grad is None:
    return res
  g = octree_depad(grad, oct, depth - 1) if padded else grad
  return res, dw_backward(g, W, s.table, s.in_h), dw_weight(data, g, s.table), g.sum(0)


# --------------------------------------------------------------------------
# the reference's CPU execution form, with torch CPU ops (timed baseline)
# --------------------------------------------------------------------------

class BlockGemmCPU:
  """Chunked gather -> mm -> scatter_add, as octree_conv.py:92-202 runs it on
  a CPU: the im2col buffer holds at most ``max_buffer`` elements per chunk."""

  def __init__(self, table, in_conv, max_buffer=int(2e8)):
    import torch
    self.torch = torch
    self.table = table if isinstance(table, torch.Tensor) else torch.from_numpy(table)
    self.kdim = self.table.shape[1]
    self.in_conv = in_conv
    self.buffer_n = 1
    self.buffer_h = self.table.shape[0]
    ideal = self.buffer_h * self.kdim * in_conv
    if ideal > max_buffer:
      kc = self.kdim * in_conv
      mb = max_buffer // kc * kc
      self.buffer_n = (ideal + mb - 1) // mb
      self.buffer_h = (self.buffer_h + self.buffer_n - 1) // self.buffer_n

  def _chunks(self):
    n = self.table.shape[0]
    for i in range(self.buffer_n):
      s = i * self.buffer_h
      e = min(n, s + self.buffer_h)
      if s < e:
        yield s, e

  def _col(self, data, s, e):
    t = self.table[s:e]
    valid = t >= 0
    buf = data.new_zeros((e - s, self.kdim, self.in_conv))
    buf[valid] = data[t[valid]]
    return buf

  def forward(self, data, W):
    out = data.new_zeros((self.table.shape[0], W.shape[2]))
    for s, e in self._chunks():
      out[s:e] = self.torch.mm(self._col(data, s, e).flatten(1, 2), W.flatten(0, 1))
    return out

  def backward(self, grad, W, rows_in):
    out = grad.new_zeros((rows_in, W.shape[1]))
    for s, e in self._chunks():
      buf = self.torch.mm(grad[s:e], W.flatten(0, 1).t()).view(-1, self.kdim, self.in_conv)
      t = self.table[s:e]
      valid = t >= 0
      src = buf[valid]
      index = t[valid].unsqueeze(-1).expand_as(src)
      out.scatter_add_(0, index, src)
    return out

  def weight(self, data, grad, W_shape):
    out = data.new_zeros(W_shape).flatten(0, 1)
    for s, e in self._chunks():
      out.addmm_(self._col(data, s, e).flatten(1, 2).t(), grad[s:e])
    return out.view(W_shape)
