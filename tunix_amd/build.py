"""Builds the HIP library (libtmx.so) in-tree for gfx950 with hipcc."""
import concurrent.futures
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, 'csrc')
OBJ = os.path.join(_HERE, 'build')
LIB_PATH = os.path.join(_HERE, 'libtmx.so')

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
    '-Wno-pass-failed',
    # keep the compiler from forming packed-fp32 VALU ops
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]


def sources():
  return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith('.hip'))


def _run(cmd):
  res = subprocess.run(cmd, capture_output=True, text=True)
  out = '\n'.join(l for l in (res.stdout + res.stderr).splitlines() if 'packed-fp32-ops' not in l)
  if res.returncode != 0:
    raise RuntimeError('hipcc failed: ' + ' '.join(cmd) + '\n' + out)
  return out


def build(verbose=False, jobs=6):
  """Compiles every .hip source under csrc/ (one object each, in parallel) into one shared library."""
  hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
  os.makedirs(OBJ, exist_ok=True)
  inc = ['-I', os.path.join(_HERE, '..', 'include')]
  srcs = sources()
  objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + '.o') for s in srcs]
  with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
    outs = list(ex.map(lambda so: _run([hipcc] + HIPCC_FLAGS + inc + ['-c', so[0], '-o', so[1]]),
                       zip(srcs, objs)))
  outs.append(_run([hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-Wl,--no-undefined', '-o', LIB_PATH] + objs))
  if verbose:
    print('\n'.join(o for o in outs if o.strip()))
  return LIB_PATH


if __name__ == '__main__':
  print(build(verbose=True))
