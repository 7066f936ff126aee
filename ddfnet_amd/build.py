"""Builds ``libddf_hip.so`` (the C-ABI DDF library) for gfx950 with hipcc, and
the PyTorch C++ extension ``_C`` on top of it.

Every ``csrc/*.hip`` file is one translation unit; they compile in parallel and
link into ``ddfnet_amd/libddf_hip.so`` next to this file, so the built library
travels with the source tree.  ``csrc/torch/ddf_torch.cpp`` (host code only) is
compiled against torch's headers into ``ddfnet_amd/_C<EXT_SUFFIX>`` and links
the library by a relative run path.  Run ``python -m ddfnet_amd.build``.
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


def torch_extension_path():
    import sysconfig
    return os.path.join(HERE, '_C' + sysconfig.get_config_var('EXT_SUFFIX'))


def build_torch_extension(verbose=True):
    """Compile the C++ autograd front end (no device code) and link it against
    torch and ``libddf_hip.so``.  Needs the library built first."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    src = os.path.join(CSRC, 'torch', 'ddf_torch.cpp')
    out = torch_extension_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), 'lib')
    rocm = os.environ.get('ROCM_PATH', '/opt/rocm')
    cmd = [os.environ.get('CXX', 'g++'), '-O2', '-fPIC', '-shared', '-std=c++17', '-w',
           '-D__HIP_PLATFORM_AMD__=1', '-DUSE_ROCM=1', '-DTORCH_EXTENSION_NAME=_C',
           '-DTORCH_API_INCLUDE_EXTENSION_H',
           '-D_GLIBCXX_USE_CXX11_ABI=%d' % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    cmd += ['-I' + p for p in cpp_extension.include_paths()]
    cmd += ['-I' + sysconfig.get_paths()['include'], '-I' + os.path.join(rocm, 'include'),
            '-I' + os.path.join(ROOT, 'include'), src, '-o', out + '.tmp',
            '-L' + torch_lib, '-L' + HERE, '-lddf_hip', '-lc10', '-lc10_hip', '-ltorch_cpu',
            '-ltorch_hip', '-ltorch', '-ltorch_python',
            '-Wl,-rpath,$ORIGIN', '-Wl,-rpath,' + torch_lib]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError('building the torch extension failed:\n' + proc.stdout)
    os.replace(out + '.tmp', out)
    if verbose:
        print('built', out)
    return out


if __name__ == '__main__':
    build(extra_flags=sys.argv[1:])
    build_torch_extension()
