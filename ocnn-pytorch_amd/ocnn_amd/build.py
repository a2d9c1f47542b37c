"""Builds libocnn_hip.so (gfx950) from csrc/ with hipcc, in-tree."""

import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(HERE, 'csrc')
LIB_DIR = os.path.join(HERE, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libocnn_hip.so')
# measurement probes (MFMA and LDS rates of the part), used by bench.py only: a library of their own
PROBE_LIB_PATH = os.path.join(LIB_DIR, 'libocnn_probe.so')
INCLUDE = os.path.join(ROOT, 'include')

# file -> extra flags.  The key/build kernels must round every fp32 operation
# separately to reproduce the reference's point normalisation bit for bit.
SOURCES = {
    'morton.hip': ['-ffp-contract=off'],
    'build.hip': ['-ffp-contract=off'],
    'neigh.hip': [],
    'conv.hip': [],
    'conv_staged.hip': [],
    'conv_rw.hip': [],
    'conv_wide.hip': [],
    'conv_sparse.hip': [],
    'wgrad_sparse.hip': [],
    'dense_rw.hip': [],
    'dw_planned.hip': [],
    'wgrad_planned.hip': [],
    'plan.hip': [],
    'misc.hip': [],
    'select.hip': [],
    'interp.hip': ['-ffp-contract=off'],
    'norm.hip': ['-ffp-contract=off'],
}

COMMON = ['-O3', '--offload-arch=gfx950', '-fPIC', '-std=c++17', '-I', INCLUDE, '-I', CSRC,
          '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']


def _hipcc():
  for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
    if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
      return cand
  raise RuntimeError('hipcc not found')


def _run(cmd):
  res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
  if res.returncode != 0:
    raise RuntimeError('command failed: {}\n{}'.format(' '.join(cmd), res.stdout))
  return res.stdout


def build_library(verbose=False):
  """Compiles every HIP source and links the shared library.  Always compiles."""
  os.makedirs(LIB_DIR, exist_ok=True)
  obj_dir = os.path.join(LIB_DIR, 'obj')
  os.makedirs(obj_dir, exist_ok=True)
  hipcc = _hipcc()

  def compile_one(item):
    name, extra = item
    obj = os.path.join(obj_dir, name.replace('.hip', '.o'))
    _run([hipcc] + COMMON + extra + ['-c', os.path.join(CSRC, name), '-o', obj])
    return obj

  with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
    objs = list(pool.map(compile_one, SOURCES.items()))
  _run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', LIB_PATH] + objs)
  _run([hipcc] + COMMON + ['-shared', os.path.join(CSRC, 'probe.hip'), '-o', PROBE_LIB_PATH])
  if verbose:
    print('built', LIB_PATH)
  return LIB_PATH


if __name__ == '__main__':
  build_library(verbose=True)
