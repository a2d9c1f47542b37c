"""ctypes binding of libocnn_hip.so (the C ABI declared in include/ocnn_hip.h).

There is no CPU fallback: if the library cannot be loaded the package raises.
"""

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_void_p, POINTER

import torch

from . import build as _build

_i, _l, _p, _f, _d = c_int, c_int64, c_void_p, c_float, c_double

# name -> (restype, argtypes); mirrors include/ocnn_hip.h one to one
SIGNATURES = {
    'ocnn_last_error': (c_char_p, []),
    'ocnn_abi_version': (_i, []),
    'ocnn_xyz2key': (_i, [_p, _p, _p, _p, _l, _i, _p, _p]),
    'ocnn_key2xyz': (_i, [_p, _l, _i, _p, _p, _p, _p, _p]),
    'ocnn_points2key': (_i, [_p, _l, POINTER(_f), _f, _p, _i, _i, _p, _p, _p]),
    'ocnn_host_encode_key': (_l, [_l, _l, _l, _l, _i]),
    'ocnn_host_decode_key': (None, [_l, _i, POINTER(_l)]),
    'ocnn_build_level_workspace_bytes': (_l, [_l]),
    'ocnn_octree_build_workspace_bytes': (_l, [_l, _i, _i, _i]),
    'ocnn_octree_build_scan': (_i, [_p, _l, _i, _i, _i, _p, _l, _p, _p, _p]),
    'ocnn_octree_build_fill': (_i, [_p, _l, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p]),
    'ocnn_build_full_layer': (_i, [_i, _i, _i, _p, _p, _p]),
    'ocnn_split_children': (_i, [_p, _l, _p, _l, _p, _p, _p]),
    'ocnn_grow_layer': (_i, [_p, _p, _l, _p, _p, _p]),
    'ocnn_leaf_average': (_i, [_p, _i, _p, _p, _l, _i, _p, _p]),
    'ocnn_leaf_points_normals': (_i, [_p, _p, _p, _p, _l, _p, _p, _p]),
    'ocnn_neigh_full': (_i, [_i, _i, _p, _p, _p]),
    'ocnn_neigh_from_parent': (_i, [_p, _p, _p, _l, _p, _p, _p]),
    'ocnn_neigh_all': (_i, [_i, _i, _i, _p, _p, _p, _p, _p, _p]),
    'ocnn_host_child_slot_lut': (None, [_i, _i, POINTER(_i), POINTER(_i)]),
    'ocnn_nempty_index': (_i, [_p, _l, _p, _p, _p]),
    'ocnn_neigh_select': (_i, [_p, _p, _i, _p, POINTER(_i), _i, _l, _p, _p, _p]),
    'ocnn_table_to_i64': (_i, [_p, _l, _p, _p]),
    'ocnn_table_to_i32': (_i, [_p, _l, _p, _p]),
    'ocnn_table_transpose': (_i, [_p, _l, _i, _l, _p, _p]),
    'ocnn_conv_workspace_bytes': (_l, [_i, _i, _i]),
    'ocnn_conv_gather_workspace_bytes': (_l, [_i, _l, _i, _i, _i]),
    'ocnn_conv_gather': (_i, [_i, _p, _l, _p, _l, _i, _p, _i, _i, _i, _i, _p, _p, _p, _l, _p]),
    'ocnn_conv_gather_choose': (_i, [_i, _l, _l, _i, _i, _i, _i, _i, _i, _l, _d, _d]),
    'ocnn_conv_wgrad_choose': (_i, [_i, _l, _l, _i, _i, _i, _i, _i, _i, _l, _d]),
    'ocnn_tile_plan_rows': (_i, []),
    'ocnn_tile_plan_count': (_i, [_p, _l, _i, _p, _p, _p]),
    'ocnn_tile_plan_offsets': (_i, [_p, _p, _l, _i, _p, _p, _p]),
    'ocnn_tile_plan_fill': (_i, [_p, _l, _i, _p, _p, _p, _p]),
    'ocnn_tile_plan_build': (_i, [_p, _l, _i, _i, _p, _p, _p, _p, _p]),
    'ocnn_tile_plan_compact': (_i, [_p, _p, _p, _i, _i, _p, _p, _p, _i, _l, _p]),
    'ocnn_conv_gather_planned_supported': (_i, [_i, _l, _i, _i]),
    'ocnn_conv_gather_planned': (_i, [_i, _p, _l, _p, _p, _p, _l, _i, _p, _i, _i, _i, _i, _p, _p,
                                      _p, _l, _p]),
    'ocnn_conv_gather_rw_supported': (_i, [_i, _l, _i, _i, _i, _i]),
    'ocnn_conv_gather_rw': (_i, [_i, _p, _l, _p, _p, _p, _i, _l, _l, _i, _p, _i, _i, _i, _i, _p, _p,
                                 _p, _l, _p]),
    'ocnn_conv_gather_rw_static_max_weight_bytes': (_l, []),
    'ocnn_conv_gather_rw_static': (_i, [_i, _p, _l, _p, _p, _p, _i, _l, _l, _i, _p, _i, _i, _i, _i, _p, _p,
                                        _p]),
    'ocnn_conv_gather_wide_supported': (_i, [_i, _l, _i, _i, _i, _i]),
    'ocnn_pair_plan_slot_counts': (_i, [_p, _l, _i, _p, _p]),
    'ocnn_pair_plan_lists': (_i, [_i, _p, _p, _p, _p, _p]),
    'ocnn_pair_plan_count': (_i, [_p, _l, _i, _p, _i, _p, _p]),
    'ocnn_pair_plan_fill': (_i, [_p, _l, _i, _p, _i, _p, _p, _p]),
    'ocnn_conv_wgrad_sparse_supported': (_i, [_i, _l, _l, _i, _i, _i, _i]),
    'ocnn_conv_wgrad_sparse_workspace_bytes': (_l, [_l, _i, _i]),
    'ocnn_conv_wgrad_sparse': (_i, [_i, _p, _l, _i, _p, _l, _i, _p, _p, _i, _l, _p, _p, _l, _p, _p, _i, _i, _i, _p,
                                    _p, _l, _p]),
    'ocnn_conv_gather_sparse_supported': (_i, [_i, _l, _i, _i, _i, _i]),
    'ocnn_conv_gather_sparse_workspace_bytes': (_l, [_i, _i]),
    'ocnn_conv_gather_sparse': (_i, [_i, _p, _l, _p, _p, _i, _l, _p, _p, _l, _i, _p, _i, _p, _l, _i, _p, _i, _i, _i,
                                     _i, _p, _p, _p, _l, _p]),
    'ocnn_conv_gather_wide': (_i, [_i, _p, _l, _p, _p, _p, _i, _l, _d, _l, _i, _p, _i, _i, _i, _i, _p, _p,
                                   _p, _l, _p]),
    'ocnn_conv_dense_supported': (_i, [_i, _l, _i, _i]),
    'ocnn_conv_dense': (_i, [_i, _p, _l, _p, _i, _i, _i, _p, _p, _p, _l, _p]),
    'ocnn_conv_dense_rw_supported': (_i, [_i, _l, _i, _i]),
    'ocnn_conv_dense_rw': (_i, [_i, _p, _l, _p, _i, _i, _i, _p, _p, _p, _l, _p]),
    'ocnn_conv_dense_wgrad_rw_supported': (_i, [_i, _l, _i, _i]),
    'ocnn_conv_dense_wgrad_rw_workspace_bytes': (_l, [_i, _i]),
    'ocnn_conv_dense_wgrad_rw': (_i, [_i, _p, _p, _l, _i, _i, _i, _p, _p, _l, _p]),
    'ocnn_conv_dense_rw_indexed': (_i, [_i, _p, _l, _p, _l, _p, _i, _i, _i, _p, _p, _l, _p, _p, _l, _p]),
    'ocnn_conv_dense_wgrad_rw_indexed': (_i, [_i, _p, _l, _p, _p, _l, _p, _l, _i, _i, _i, _p, _p, _l, _p]),
    'ocnn_conv_wgrad_workspace_bytes': (_l, [_l, _i, _i, _i]),
    'ocnn_conv_wgrad_workspace_bytes_for': (_l, [_i, _l, _l, _i, _i, _i]),
    'ocnn_conv_wgrad': (_i, [_i, _p, _l, _p, _p, _l, _i, _i, _i, _i, _p, _p, _l, _p]),
    'ocnn_conv_wgrad_planned_supported': (_i, [_i, _l, _l, _i, _i, _i, _i]),
    'ocnn_conv_wgrad_planned_workspace_bytes': (_l, [_i, _i, _i]),
    'ocnn_conv_wgrad_planned_workspace_bytes_for': (_l, [_i, _l, _l, _i, _i, _i]),
    'ocnn_conv_wgrad_planned': (_i, [_i, _p, _l, _p, _p, _p, _p, _i, _l, _l, _i, _i, _i, _i, _p, _p,
                                     _l, _p]),
    'ocnn_dwconv_gather': (_i, [_i, _p, _l, _p, _l, _i, _p, _i, _i, _p, _p, _p]),
    'ocnn_dwconv_gather_planned_supported': (_i, [_i, _l, _i, _i, _i]),
    'ocnn_dwconv_gather_planned': (_i, [_i, _p, _l, _p, _p, _p, _i, _l, _l, _i, _p, _i, _i, _p, _p, _p]),
    'ocnn_dwconv_wgrad_planned_supported': (_i, [_i, _l, _l, _i, _i, _i]),
    'ocnn_dwconv_wgrad_planned_workspace_bytes': (_l, [_i, _i]),
    'ocnn_dwconv_wgrad_planned': (_i, [_i, _p, _l, _p, _p, _p, _p, _i, _l, _l, _i, _i, _p, _p, _l, _p]),
    'ocnn_batch_norm_supported': (_i, [_i, _l, _i]),
    'ocnn_batch_norm_workspace_bytes': (_l, [_i]),
    'ocnn_batch_norm_stats': (_i, [_i, _p, _l, _i, _f, _p, _p, _p, _p, _p, _i, _f, _p, _p, _l, _p]),
    'ocnn_batch_norm_apply': (_i, [_i, _p, _l, _i, _p, _p, _p, _p, _i, _i, _p, _p, _p]),
    'ocnn_batch_norm_backward': (_i, [_i, _p, _p, _l, _i, _p, _p, _p, _p, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p,
                                      _p, _l, _p]),
    'ocnn_search_key': (_i, [_p, _l, _p, _l, _p, _p]),
    'ocnn_search_points': (_i, [_p, _l, _i, _p, _l, _i, _p, _p]),
    'ocnn_interp_linear_prepare': (_i, [_p, _l, _i, _p, _l, _i, _p, _p, _p, _p]),
    'ocnn_locate_points': (_i, [_p, _l, _p, _i, _i, _i, _i, _i, _p, _p]),
    'ocnn_interp_linear_locate': (_i, [_p, _l, _p, _i, _i, _i, _i, _i, _p, _p, _p, _p]),
    'ocnn_csr_rows': (_i, [_i, _p, _i, _p, _p, _p, _i, _p, _p, _l, _p]),
    'ocnn_csr_transpose_workspace_bytes': (_l, [_l]),
    'ocnn_csr_transpose': (_i, [_p, _p, _p, _l, _i, _l, _p, _l, _p, _p, _p, _p]),
    'ocnn_max_pool': (_i, [_i, _p, _p, _p, _l, _i, _p, _p, _p]),
    'ocnn_max_unpool': (_i, [_i, _p, _p, _p, _p, _l, _i, _p, _p]),
    'ocnn_max_gather': (_i, [_i, _p, _p, _p, _l, _i, _p, _p]),
    'ocnn_dwconv_wgrad_workspace_bytes': (_l, [_l, _i, _i]),
    'ocnn_dwconv_wgrad': (_i, [_i, _p, _l, _p, _p, _l, _i, _i, _p, _p, _l, _p]),
    'ocnn_pad': (_i, [_i, _p, _p, _l, _i, _f, _p, _p]),
    'ocnn_depad': (_i, [_i, _p, _p, _l, _i, _p, _p]),
    'ocnn_colsum_workspace_bytes': (_l, [_l, _i]),
    'ocnn_colsum': (_i, [_i, _p, _l, _i, _p, _p, _l, _p]),
}

_lib = None


def lib():
  """Loads the library once.  A library that is missing, or that was built from other sources
  than the ones in csrc/ and include/ now (their hash is stored beside it), is built first: a
  stale binary is never loaded."""
  global _lib
  if _lib is not None:
    return _lib
  path = _build.LIB_PATH
  if not _build.is_current():
    _build.build_library()
  handle = ctypes.CDLL(path)
  for name, (res, args) in SIGNATURES.items():
    fn = getattr(handle, name)      # AttributeError if the symbol is missing
    fn.restype = res
    fn.argtypes = args
  _lib = handle
  return _lib


class OcnnHipError(RuntimeError):
  pass


def check(rc):
  if rc != 0:
    raise OcnnHipError('libocnn_hip: {} (code {})'.format(
        lib().ocnn_last_error().decode('utf-8', 'replace'), rc))


DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

# codes of ocnn_conv_gather_choose / ocnn_conv_wgrad_choose (include/ocnn_hip.h)
(GATHER_PLAIN, GATHER_DENSE_RW, GATHER_DENSE, GATHER_RW, GATHER_SPARSE, GATHER_WIDE, GATHER_PLANNED,
 GATHER_ZERO_PADDED) = range(8)
WGRAD_PLAIN, WGRAD_DENSE_RW, WGRAD_SPARSE, WGRAD_PLANNED, WGRAD_ZERO_PADDED = range(5)


def dtype_code(t):
  try:
    return DTYPE_CODE[t.dtype]
  except KeyError:
    raise TypeError('unsupported feature dtype {}; use float32, float16 or bfloat16'.format(t.dtype))


def require_gpu(*tensors):
  """The kernels run on the GPU only; anything else is an error, not a fallback."""
  for t in tensors:
    if t is not None and not t.is_cuda:
      raise RuntimeError('ocnn_amd kernels need tensors on a HIP device, got a tensor on '
                         '{}'.format(t.device))


def ptr(t):
  return None if t is None else t.data_ptr()


def _raw_stream_fast():
  return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _raw_stream_public():
  return torch.cuda.current_stream().cuda_stream


def stream():
  """The current HIP stream of the current device as an integer handle.  (The public route,
  torch.cuda.current_stream(), builds a Stream object through several layers of Python: 15 us a
  call, a third of the host time of a layer's forward + backward; the two calls it ends in are
  taken directly where torch has them.)"""
  global stream
  try:
    handle = _raw_stream_fast()
    stream = _raw_stream_fast
  except (AttributeError, RuntimeError, TypeError):
    handle = _raw_stream_public()
    stream = _raw_stream_public
  return handle


def workspace(nbytes, device):
  return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
