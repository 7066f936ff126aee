"""Builds ``libddf_hip.so`` (the C-ABI DDF library) for gfx950 with hipcc.

Every ``csrc/*.hip`` file is one translation unit; they compile in parallel and
link into ``ddfnet_amd/libddf_hip.so`` next to this file, so the built library
travels with the source tree.  Run ``python -m ddfnet_amd.build``.
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, 'csrc')
OBJ_DIR = os.path.join(HERE, 'build')
LIB_PATH = os.path.join(HERE, 'libddf_hip.so')

ARCH = 'gfx950'
# Packed fp32 VALU forms are switched off for every device function.
HIPCC_FLAGS = [
    '--offload-arch=' + ARCH, '-O3', '-fPIC', '-std=c++17', '-Wall',
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    '-I' + os.path.join(ROOT, 'include'), '-I' + CSRC,
]


def hipcc():
    for cand in (os.environ.get('HIPCC'), '/opt/rocm/bin/hipcc', 'hipcc'):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError('hipcc not found')


def _compile(src, extra):
    obj = os.path.join(OBJ_DIR, os.path.basename(src).replace('.hip', '.o'))
    cmd = [hipcc()] + HIPCC_FLAGS + list(extra) + ['-c', src, '-o', obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError('hipcc failed on %s:\n%s' % (src, proc.stdout))
    return obj, proc.stdout


def build(verbose=True, extra_flags=(), jobs=None):
    """Compile every HIP source and link the shared library.  Always
    recompiles, so a stale object can never pass for a successful build."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, '*.hip')))
    if not sources:
        raise RuntimeError('no HIP sources under ' + CSRC)
    jobs = jobs or min(len(sources), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda s: _compile(s, extra_flags), sources))
    objs = [o for o, _ in results]
    if verbose:
        for (_, log), src in zip(results, sources):
            log = '\n'.join(l for l in log.splitlines()
                            if 'packed-fp32-ops' not in l and l.strip())
            if log:
                print('[%s]\n%s' % (os.path.basename(src), log))
    tmp = LIB_PATH + '.tmp'
    cmd = [hipcc(), '--offload-arch=' + ARCH, '-shared', '-fPIC', '-o', tmp] + objs
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError('link failed:\n' + proc.stdout)
    os.replace(tmp, LIB_PATH)
    if verbose:
        print('built', LIB_PATH)
    return LIB_PATH


if __name__ == '__main__':
    build(extra_flags=sys.argv[1:])
