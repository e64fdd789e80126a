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


# The host side of the same sources (argument checks, launch planning, workspace carving) instrumented with
# AddressSanitizer and UndefinedBehaviorSanitizer; the device code is compiled as usual (sanitizers on
# host code only).  Loaded by a CPU test in a child process that preloads the sanitizer runtime.
HOSTSAN_LIB_PATH = os.path.join(_HERE, 'libtmx_hostsan.so')
HOSTSAN_OBJ = os.path.join(_HERE, 'build_hostsan')
HOSTSAN_FLAGS = ['-Xarch_host', '-fsanitize=address', '-Xarch_host', '-fsanitize=undefined',
                 '-Xarch_host', '-fno-omit-frame-pointer', '-Xarch_host', '-fno-sanitize-recover=undefined']


def build(verbose=False, jobs=6, host_sanitizers=False):
  """Compiles every .hip source under csrc/ (one object each, in parallel) into one shared library."""
  hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
  obj_dir, lib_path = (HOSTSAN_OBJ, HOSTSAN_LIB_PATH) if host_sanitizers else (OBJ, LIB_PATH)
  extra = HOSTSAN_FLAGS if host_sanitizers else []
  os.makedirs(obj_dir, exist_ok=True)
  inc = ['-I', os.path.join(_HERE, '..', 'include')]
  srcs = sources()
  objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + '.o') for s in srcs]
  with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
    outs = list(ex.map(lambda so: _run([hipcc] + HIPCC_FLAGS + extra + inc + ['-c', so[0], '-o', so[1]]),
                       zip(srcs, objs)))
  link = [hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', lib_path]
  # the sanitizer runtime is supplied by the loading process (preloaded), so its symbols stay undefined here
  link += ['-shared-libsan', '-fsanitize=address', '-fsanitize=undefined'] if host_sanitizers else ['-Wl,--no-undefined']
  outs.append(_run(link + objs))
  if verbose:
    print('\n'.join(o for o in outs if o.strip()))
  return lib_path


def sanitizer_runtime():
  """Path of clang's shared AddressSanitizer runtime (what a process that loads the host-sanitizer
  build has to preload), or None."""
  hipcc = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
  res = subprocess.run([hipcc, '-print-file-name=libclang_rt.asan-x86_64.so'], capture_output=True, text=True)
  path = res.stdout.strip()
  return path if res.returncode == 0 and os.path.isabs(path) and os.path.exists(path) else None


if __name__ == '__main__':
  import sys
  print(build(verbose=True, host_sanitizers='--host-sanitizers' in sys.argv))
