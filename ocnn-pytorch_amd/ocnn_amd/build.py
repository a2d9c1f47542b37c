"""Builds libocnn_hip.so (gfx950) from csrc/ with hipcc, in-tree."""

import hashlib
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(HERE, 'csrc')
LIB_DIR = os.path.join(HERE, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libocnn_hip.so')
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


STAMP_PATH = os.path.join(LIB_DIR, 'sources.sha256')


def source_hash():
  """Hash of everything the library is built from (sources, headers, flags)."""
  h = hashlib.sha256()
  names = sorted(os.listdir(CSRC))
  for path in [os.path.join(CSRC, n) for n in names] + [os.path.join(INCLUDE, n) for n in sorted(os.listdir(INCLUDE))]:
    if os.path.isfile(path):
      h.update(os.path.basename(path).encode())
      with open(path, 'rb') as f:
        h.update(f.read())
  h.update(repr((COMMON[:4] + COMMON[8:], sorted(SOURCES.items()))).encode())
  return h.hexdigest()


def is_current():
  """True when the library exists and was built from the sources as they are now."""
  try:
    with open(STAMP_PATH) as f:
      stamp = f.read().strip()
  except OSError:
    return False
  return os.path.exists(LIB_PATH) and stamp == source_hash()


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
  with open(STAMP_PATH, 'w') as f:
    f.write(source_hash() + '\n')
  if verbose:
    print('built', LIB_PATH)
  return LIB_PATH


if __name__ == '__main__':
  build_library(verbose=True)
