"""Builds libqwix_hip.so (gfx950) from the .hip sources in this directory with hipcc.

Run directly (`python qwix_amd/csrc/build.py`) or through `__graft_entry__.build()`.
Each source is compiled to an object file in `build/`, then everything is linked into
`qwix_amd/libqwix_hip.so`, which the ctypes loader in `qwix_amd/_lib.py` opens.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OUT = os.path.join(PKG, 'libqwix_hip.so')
OBJ_DIR = os.path.join(HERE, 'build')
HIPCC = os.environ.get('HIPCC', '/opt/rocm/bin/hipcc')
FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-fvisibility=hidden',
    # No packed-FP32 VALU ops (v_pk_*_f32) in generated code.
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-Wno-unused-command-line-argument',
]


def sources():
  return sorted(f for f in os.listdir(HERE) if f.endswith('.hip'))


def _compile(src: str, force: bool) -> str:
  obj = os.path.join(OBJ_DIR, src[:-4] + '.o')
  deps = [os.path.join(HERE, src), os.path.join(HERE, 'common.h'),
          os.path.join(os.path.dirname(PKG), 'include', 'qwix_hip.h')]
  if not force and os.path.exists(obj) and all(os.path.getmtime(obj) > os.path.getmtime(d) for d in deps):
    return obj
  cmd = [HIPCC, *FLAGS, '-c', os.path.join(HERE, src), '-o', obj]
  r = subprocess.run(cmd, capture_output=True, text=True)
  err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
  if r.returncode != 0:
    raise RuntimeError(f'hipcc failed on {src}:\n{err}')
  if err.strip():
    print(err, file=sys.stderr)
  return obj


def build(force: bool = True, verbose: bool = True) -> str:
  os.makedirs(OBJ_DIR, exist_ok=True)
  srcs = sources()
  with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
    objs = list(ex.map(lambda s: _compile(s, force), srcs))
  cmd = [HIPCC, '--offload-arch=gfx950', '-shared', '-fPIC', *objs, '-o', OUT]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f'link failed:\n{r.stderr}')
  if verbose:
    print(f'built {OUT} from {len(srcs)} sources')
  return OUT


if __name__ == '__main__':
  build(force='--incremental' not in sys.argv)
