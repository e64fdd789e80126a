"""Builds the HIP library (libtmx.so) in-tree for gfx950 with hipcc."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, 'csrc')
LIB_PATH = os.path.join(_HERE, 'libtmx.so')

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-shared',
    '-Wno-pass-failed',
    # keep the compiler from forming packed-fp32 VALU ops
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]


def sources():
  return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith('.hip'))


def build(verbose=False):
  """Compiles every .hip source under csrc/ into one shared library."""
  hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
  cmd = [hipcc] + HIPCC_FLAGS + ['-I', os.path.join(_HERE, '..', 'include'), '-o', LIB_PATH] + sources()
  res = subprocess.run(cmd, capture_output=True, text=True)
  out = '\n'.join(l for l in (res.stdout + res.stderr).splitlines() if 'packed-fp32-ops' not in l)
  if verbose and out.strip():
    print(out)
  if res.returncode != 0:
    raise RuntimeError('hipcc failed:\n' + out)
  return LIB_PATH


if __name__ == '__main__':
  print(build(verbose=True))
