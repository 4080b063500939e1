"""Builds libhidet_qmm.so from the HIP sources under csrc/ with hipcc for gfx950.

Plays the part of the reference's compile step for these operators (python/hidet/backend/build.py:206-280,
`HIPCC.compile`): same compiler, same `--offload-arch`, `-fPIC --shared`; `-ffast-math` is dropped because
the quantization kernels must divide and round exactly.
"""
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB_DIR = os.path.join(HERE, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libhidet_qmm.so')
ARCH = 'gfx950'

FLAGS = [
    '--offload-arch=' + ARCH, '-O3', '-std=c++17', '-fPIC', '-fvisibility=hidden',
    # keep the compiler from forming packed-fp32 instructions
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # kernel arguments arrive in scalar registers with the wave instead of being fetched by its first instructions
    # (a kernel's first load waits about 0.3 us less; the code falls back to fetching them where that is not supported)
    '-mllvm', '-amdgpu-kernarg-preload-count=16',
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith('.hip'))


def hipcc():
    exe = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(exe):
        raise RuntimeError('hipcc not found: the kernels can only be built with ROCm installed')
    return exe


def _compile(src, obj, verbose):
    cmd = [hipcc()] + FLAGS + ['-c', os.path.join(CSRC, src), '-o', obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = '\n'.join(l for l in r.stdout.splitlines() if 'packed-fp32-ops' not in l)
    if r.returncode != 0:
        raise RuntimeError('hipcc failed on {}:\n{}'.format(src, out))
    if verbose and out.strip():
        print(out, file=sys.stderr)


def build(verbose=False, jobs=8):
    """Compile every .hip source and link the shared library (always recompiles)."""
    obj_dir = os.path.join(HERE, 'build')
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(obj_dir, s[:-4] + '.o') for s in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _compile(so[0], so[1], verbose), zip(srcs, objs)))
    tmp = LIB_PATH + '.tmp'
    cmd = [hipcc(), '--offload-arch=' + ARCH, '-shared', '-fPIC', '-o', tmp] + objs
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError('link failed:\n' + r.stdout)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == '__main__':
    print(build(verbose=True))
