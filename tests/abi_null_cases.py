"""Calls every launching entry point of libocnn_hip.so with valid sizes and bad pointers, bad sizes
or no workspace, and prints what came back as JSON.  Run as a child process by
tests/test_abi_host.py with every GPU hidden: an entry point that lets such a call through then
fails to launch (no device) instead of faulting a GPU.

A case lists the arguments in the order of the C signature: numbers are valid sizes; 'P' is a
required device pointer, 'O' an optional one (always passed as NULL), 'W' the workspace size, and a
list is the content of a required host array (host arrays are real memory: the library reads them).
"""

import ctypes
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, 'ocnn-pytorch_amd'))

FAKE = 0x7f0000001000          # a non-null value that is never dereferenced on the host
BIG = 1 << 40
F = [FAKE] * 8                 # a host array of device pointers

CASES = {
    'ocnn_xyz2key': ['P', 'P', 'P', 'O', 10, 5, 'P', 'O'],
    'ocnn_key2xyz': ['P', 10, 5, 'P', 'P', 'P', 'P', 'O'],
    'ocnn_points2key': ['P', 10, [-1.0, -1.0, -1.0], 16.0, 'O', 0, 5, 'P', 'P', 'O'],
    'ocnn_octree_build_scan': ['P', 10, 3, 2, 0, 'P', 'W', 'P', 'P', 'O'],
    'ocnn_octree_build_fill': ['P', 10, 3, 2, 1, 0, [8, 1], 'P', F, F, 'P', 'P', 'O'],
    'ocnn_build_full_layer': [2, 1, 1, 'P', 'P', 'O'],
    'ocnn_split_children': ['P', 10, 'P', 'W', 'P', 'P', 'O'],
    'ocnn_grow_layer': ['P', 'P', 4, 'P', 'P', 'O'],
    'ocnn_leaf_average': ['P', 3, 'P', 'P', 4, 0, 'P', 'O'],
    'ocnn_leaf_points_normals': ['P', 'P', 'P', 'P', 4, 'P', 'P', 'O'],
    'ocnn_neigh_full': [2, 1, 'O', 'P', 'O'],
    'ocnn_neigh_from_parent': ['P', 'P', 'P', 4, 'O', 'P', 'O'],
    'ocnn_neigh_all': [3, 2, 1, [1, 8, 64, 64], [1, 8, 8, 8], F, F, F, 'O'],
    'ocnn_nempty_index': ['P', 10, 'P', 'O', 'O'],
    'ocnn_neigh_select': ['P', 'O', 1, 'O', 'O', 27, 10, 'O', 'P', 'O'],
    'ocnn_table_to_i64': ['P', 10, 'P', 'O'],
    'ocnn_table_to_i32': ['P', 10, 'P', 'O'],
    'ocnn_table_transpose': ['P', 10, 27, 10, 'P', 'O'],
    'ocnn_conv_gather': [2, 'P', 200, 'P', 200, 27, 'P', 64, 64, 0, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_tile_plan_count': ['P', 200, 27, 'P', 'O', 'O'],
    'ocnn_tile_plan_offsets': ['P', 'P', 2, 416, 'P', 'P', 'O'],
    'ocnn_tile_plan_fill': ['P', 200, 27, 'P', 'P', 'P', 'O'],
    'ocnn_tile_plan_build': ['P', 200, 27, 512, 'P', 'O', 'P', 'P', 'O'],
    'ocnn_tile_plan_compact': ['P', 'P', 'P', 416, 512, 'P', 'P', 'P', 27, 2, 'O'],
    'ocnn_conv_gather_planned': [2, 'P', 200, 'P', 'P', 'P', 200, 27, 'P', 64, 64, 0, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_conv_gather_rw': [2, 'P', 200, 'P', 'P', 'P', 100, 150, 200, 27, 'P', 64, 64, 0, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_conv_gather_rw_static': [2, 'P', 200, 'P', 'P', 'P', 100, 150, 200, 27, 'P', 64, 64, 0, 0, 'O', 'P', 'O'],
    'ocnn_conv_gather_wide': [2, 'P', 200, 'P', 'P', 'P', 100, 150, 0.3, 200, 27, 'P', 128, 128, 0, 0, 'O', 'P', 'P',
                              'W', 'O'],
    'ocnn_pair_plan_slot_counts': ['P', 2, 27, 'P', 'O'],
    'ocnn_pair_plan_lists': [27, [5] * 27, [0] * 32, [0] * 32, [0] * 5, [0]],
    'ocnn_pair_plan_count': ['P', 2, 27, 'P', 27, 'P', 'O'],
    'ocnn_pair_plan_fill': ['P', 2, 27, 'P', 27, 'P', 'P', 'O'],
    'ocnn_conv_wgrad_sparse': [2, 'P', 200, 64, 'P', 200, 64, 'P', 'P', 100, 150, 'P', 'P', 10, list(range(27)),
                               [5] * 27, 27, 27, 1, 'P', 'P', 'W', 'O'],
    'ocnn_conv_gather_sparse': [2, 'P', 200, 'P', 'P', 100, 150, 'P', 'P', 10, 10, 'P', 27, [0, 7, 14, 21, 27], 200,
                                27, 'P', 64, 64, 0, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_conv_dense': [2, 'P', 200, 'P', 64, 128, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_conv_dense_rw': [2, 'P', 200, 'P', 64, 128, 0, 'O', 'P', 'P', 'W', 'O'],
    'ocnn_conv_dense_wgrad_rw': [2, 'P', 'P', 200, 64, 128, 0, 'P', 'P', 'W', 'O'],
    'ocnn_conv_dense_rw_indexed': [2, 'P', 200, 'O', 200, 'P', 64, 128, 0, 'O', 'P', 200, 'O', 'P', 'W', 'O'],
    'ocnn_conv_dense_wgrad_rw_indexed': [2, 'P', 200, 'O', 'P', 200, 'O', 200, 64, 128, 0, 'P', 'P', 'W', 'O'],
    'ocnn_conv_wgrad': [2, 'P', 200, 'P', 'P', 200, 27, 64, 64, 0, 'P', 'P', 'W', 'O'],
    'ocnn_conv_wgrad_planned': [2, 'P', 200, 'P', 'P', 'P', 'P', 100, 150, 200, 27, 64, 64, 0, 'P', 'P', 'W', 'O'],
    'ocnn_dwconv_gather': [2, 'P', 200, 'P', 200, 27, 'P', 64, 0, 'O', 'P', 'O'],
    'ocnn_dwconv_gather_planned': [2, 'P', 200, 'P', 'P', 'P', 100, 150, 200, 27, 'P', 64, 0, 'O', 'P', 'O'],
    'ocnn_dwconv_wgrad_planned': [2, 'P', 200, 'P', 'P', 'P', 'P', 100, 150, 200, 27, 64, 'P', 'P', 'W', 'O'],
    'ocnn_batch_norm_stats': [2, 'P', 200, 64, 1e-5, 'P', 'P', 'P', 'O', 'O', 0, 0.1, 'O', 'P', 'W', 'O'],
    'ocnn_batch_norm_apply': [2, 'P', 200, 64, 'P', 'P', 'O', 'O', 0, 1, 'O', 'P', 'O'],
    'ocnn_batch_norm_backward': [2, 'P', 'P', 200, 64, 'P', 'P', 'O', 'O', 0, 1, 1, 'O', 'O', 'O', 'P', 'P', 'O', 'O',
                                 'P', 'W', 'O'],
    'ocnn_search_key': ['P', 10, 'P', 10, 'P', 'O'],
    'ocnn_search_points': ['P', 10, 5, 'P', 10, 1, 'P', 'O'],
    'ocnn_interp_linear_prepare': ['P', 10, 5, 'P', 10, 1, 'P', 'P', 'P', 'O'],
    'ocnn_locate_points': ['P', 10, F, 3, 2, 1, 0, 1, 'P', 'O'],
    'ocnn_interp_linear_locate': ['P', 10, F, 3, 2, 1, 0, 1, 'P', 'P', 'P', 'O'],
    'ocnn_csr_rows': [0, 'O', 8, 'P', 'O', 'P', 4, 'O', 'P', 10, 'O'],
    'ocnn_csr_transpose': ['P', 'O', 'O', 10, 8, 10, 'P', 'W', 'P', 'P', 'O', 'O'],
    'ocnn_max_pool': [2, 'P', 'O', 'O', 10, 8, 'P', 'P', 'O'],
    'ocnn_max_unpool': [2, 'P', 'P', 'O', 'O', 10, 8, 'P', 'O'],
    'ocnn_max_gather': [2, 'P', 'P', 'O', 10, 8, 'P', 'O'],
    'ocnn_dwconv_wgrad': [2, 'P', 200, 'P', 'P', 200, 27, 64, 'P', 'P', 'W', 'O'],
    'ocnn_pad': [2, 'O', 'P', 10, 8, 0.0, 'P', 'O'],
    'ocnn_depad': [2, 'P', 'P', 10, 8, 'P', 'O'],
    'ocnn_colsum': [2, 'P', 10, 8, 'P', 'P', 'W', 'O'],
}

# host-only (nothing is launched): a call with good arguments succeeds
HOST_ONLY = {'ocnn_pair_plan_lists'}


def host_array(ctype, values):
  arr = (ctype * max(len(values), 64))()
  for i, v in enumerate(values):
    arr[i] = v
  return arr


def main():
  from ocnn_amd import _lib
  hip = ctypes.CDLL('libamdhip64.so')
  count = ctypes.c_int(0)
  rc = hip.hipGetDeviceCount(ctypes.byref(count))
  if rc == 0 and count.value > 0:
    print(json.dumps({'skipped': 'a GPU is visible to this process'}))
    return
  L = _lib.lib()
  # element types of the host arrays (void* host arrays hold int64 / pointers)
  elem = {('ocnn_points2key', 2): ctypes.c_float, ('ocnn_pair_plan_lists', 2): ctypes.c_int32,
          ('ocnn_pair_plan_lists', 4): ctypes.c_int32, ('ocnn_pair_plan_lists', 5): ctypes.c_int32,
          ('ocnn_conv_wgrad_sparse', 14): ctypes.c_int32, ('ocnn_conv_gather_sparse', 13): ctypes.c_int32}
  out = {}
  keep = []
  for name, spec in CASES.items():
    fn = getattr(L, name)
    argtypes = _lib.SIGNATURES[name][1]
    assert len(argtypes) == len(spec), (name, len(argtypes), len(spec))

    def build(null=(), sizes=None, ws=BIG):
      args = []
      for i, a in enumerate(spec):
        if a == 'P':
          args.append(None if i in null else FAKE)
        elif a == 'O':
          args.append(None)
        elif a == 'W':
          args.append(ws)
        elif isinstance(a, list):
          if i in null:
            args.append(None)
          else:
            arr = host_array(elem.get((name, i), ctypes.c_int64), a)
            keep.append(arr)
            args.append(arr)
        else:
          args.append(a if sizes is None or i not in sizes else sizes[i])
      return args

    def call(**kw):
      rc = fn(*build(**kw))
      return [rc, L.ocnn_last_error().decode('utf-8', 'replace') if rc != 0 else '']

    required = [i for i, a in enumerate(spec) if a == 'P' or isinstance(a, list)]
    res = {'all_null': call(null=set(required)), 'one_null': {}, 'negative': {}, 'no_workspace': None}
    for i in required:
      res['one_null'][str(i)] = call(null={i})
    for i, a in enumerate(spec):
      if argtypes[i] is ctypes.c_int64 and a != 'W':
        res['negative'][str(i)] = call(sizes={i: -1})
    if 'W' in spec:
      res['no_workspace'] = call(ws=0)
    res['good'] = call()            # no device: launches fail, nothing runs
    out[name] = res
  print(json.dumps(out))


if __name__ == '__main__':
  main()
