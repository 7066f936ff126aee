"""CPU-side checks: the C-ABI library loads and exports every symbol the header
declares, the host wrapper mirrors the reference's argument contract, and the
stock-PyTorch modules around the operator have the reference's structure.  No
kernel is launched here."""
import os
import re

import pytest
import torch

import ddfnet_amd
from ddfnet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    text = open(os.path.join(ROOT, 'include', 'ddf_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(ddf_hip_\w+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    assert ddfnet_amd.is_built(), 'run `python -m ddfnet_amd.build` first'
    lib = _lib.lib()
    names = header_functions()
    assert len(names) >= 6
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_lib.SYMBOLS) == names


def test_version_and_status_strings():
    lib = _lib.lib()
    assert lib.ddf_hip_version() >= 100
    assert lib.ddf_hip_status_string(0) == b'ok'
    assert b'workspace' in lib.ddf_hip_status_string(3)


def test_argument_validation_needs_no_gpu():
    """Bad arguments are rejected before anything touches the device."""
    lib = _lib.lib()
    assert lib.ddf_hip_forward(None, None, None, None, 1, 1, 4, 4, 2, 1, 1, 0, 1, 0, None) == 1
    assert b'kernel_size' in lib.ddf_hip_last_error()
    assert lib.ddf_hip_forward(None, None, None, None, 1, 1, 4, 4, 3, 0, 1, 0, 1, 0, None) == 1
    assert lib.ddf_hip_forward(None, None, None, None, 1, 1, 4, 4, 3, 1, 1, 2, 1, 0, None) == 1
    assert lib.ddf_hip_forward(None, None, None, None, 1, 1, 4, 4, 3, 1, 1, 0, 9, 0, None) == 1
    assert lib.ddf_hip_forward(None, None, None, None, -1, 1, 4, 4, 3, 1, 1, 0, 1, 0, None) == 1
    # empty problem: success without touching any pointer
    assert lib.ddf_hip_forward(None, None, None, None, 0, 8, 4, 4, 3, 1, 1, 0, 1, 0, None) == 0
    assert lib.ddf_hip_backward_workspace_bytes(1, 1, 4, 4, 2, 1, 1, 0, 1, 7, 0) == 0


def test_ddf_rejects_cpu_tensors_like_the_reference():
    x = torch.randn(1, 2, 4, 4)
    with pytest.raises(AssertionError, match='input feature must be a CUDA tensor'):
        ddfnet_amd.ddf(x, torch.randn(1, 2, 3, 3), torch.randn(1, 9, 4, 4))
    with pytest.raises(RuntimeError, match='not implemented on CPU'):
        ddfnet_amd.OP_DICT['mul'].forward(x, x, x, 3, 1, 1, x)


def test_public_surface_matches_reference_package():
    import ddf as dropin
    for name in ('ddf', 'DDFFunction', 'DDFPack', 'DDFUpPack', 'FilterNorm',
                 'build_spatial_branch', 'build_channel_branch', 'OP_DICT'):
        assert getattr(dropin, name) is getattr(ddfnet_amd, name)
    assert sorted(dropin.OP_DICT) == ['add', 'add_faster', 'mul', 'mul_faster']


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, '_lib', None)
    monkeypatch.setattr(_lib, 'LIB_PATH', str(tmp_path / 'libddf_hip.so'))
    with pytest.raises(_lib.DDFHipError, match='no CPU or PyTorch fallback'):
        _lib.lib()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, 'ddfnet_amd')
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(('.py', '.hip', '.h', '.cpp')):
                src = open(os.path.join(dirpath, f)).read()
                assert 'oracle' not in src, os.path.join(dirpath, f)


# ------------------------------- modules ----------------------------------
def test_filter_norm_spatial_closed_form():
    from ddfnet_amd import FilterNorm
    fn = FilterNorm(1, 3, 'spatial', 'relu')
    x = torch.arange(1., 10.).view(1, 9, 1, 1).double()
    got = fn(x).view(-1)
    std = (60.0 / 8.0) ** 0.5  # unbiased
    gain = (2.0 ** 0.5) / 3.0  # calculate_gain('relu') / kernel_size
    want = (torch.arange(1., 10.).double() - 5.0) / (std + 1e-10) * gain
    assert torch.allclose(got, want, atol=1e-12)


def test_filter_norm_channel_learned_gain_and_mean():
    from ddfnet_amd import FilterNorm
    torch.manual_seed(0)
    fn = FilterNorm(4, 3, 'channel', 'linear', running_std=True, running_mean=True)
    assert fn.std.shape == (36,) and fn.mean.shape == (36,)
    x = torch.randn(5, 36, 1, 1)
    got = fn(x)
    assert got.shape == (5, 36)
    z = x.view(5, 4, 9)
    z = (z - z.mean(2, keepdim=True)) / (z.std(2, keepdim=True) + 1e-10)
    want = z.reshape(5, 36) * fn.std[None] + fn.mean[None]
    assert torch.allclose(got, want, atol=1e-6)


@pytest.mark.parametrize('c,want', [(64, 9429), (128, 35490), (256, 137532), (512, 536175)])
def test_ddfpack_parameter_counts(c, want):
    """Per-pack parameter counts at se_ratio 0.2 that add up to the README's
    16.8 M for ddf_mul_resnet50."""
    from ddfnet_amd import DDFPack
    assert sum(p.numel() for p in DDFPack(c).parameters()) == want


def test_ddfpack_state_dict_names():
    from ddfnet_amd import DDFPack
    keys = sorted(DDFPack(16, head=2).state_dict())
    assert keys == ['channel_branch.1.bias', 'channel_branch.1.weight',
                    'channel_branch.3.bias', 'channel_branch.3.weight',
                    'channel_branch.4.std', 'spatial_branch.0.bias', 'spatial_branch.0.weight']


def test_ddfuppack_structure():
    from ddfnet_amd import DDFUpPack
    up = DDFUpPack(8, scale_factor=2)
    assert len(up.spatial_branch) == 4 and len(up.channel_branch) == 4
    assert isinstance(up.spatial_branch[0][0], torch.nn.Conv2d)  # depthwise guidance conv
    up2 = DDFUpPack(8, scale_factor=2, joint_channels=8)
    assert isinstance(up2.spatial_branch[0][1], ddfnet_amd.FilterNorm)


@pytest.mark.parametrize('name,want', [('ddf_mul_resnet50', 16843748),
                                       ('ddf_add_resnet50', 16843748),
                                       ('ddf_mul_resnet101', 28146912)])
def test_ddf_resnet_parameter_counts(name, want):
    """The reference's model table lists 16.8 M and 28.1 M parameters
    (README.md:20-23); these are the exact sums for this skeleton."""
    from ddfnet_amd import ddf_resnet
    model = getattr(ddf_resnet, name)()
    assert sum(p.numel() for p in model.parameters()) == want


def test_ddf_resnet_has_sixteen_packs():
    from ddfnet_amd import ddf_resnet, DDFPack
    model = ddf_resnet.ddf_mul_resnet50()
    packs = [m for m in model.modules() if isinstance(m, DDFPack)]
    assert len(packs) == 16
    assert [p.stride for p in packs].count(2) == 3


# ---------------------------------------------------------------------------
# host logic of the library and of bench.py (no device needed)
# ---------------------------------------------------------------------------
def test_workspace_size_is_host_arithmetic():
    """The workspace query needs no device.  At the stage-3 benchmark shape the
    filter gradients split the 256 channels 8 ways and keep the 14 rows in one
    strip: 8 partial dSF tensors in fp32, no dCF partials."""
    lib = _lib.lib()
    n_sf = 64 * 9 * 14 * 14
    assert lib.ddf_hip_backward_workspace_bytes(64, 256, 14, 14, 3, 1, 1, 0, 1, 7, 0) == 8 * n_sf * 4
    # fp16 partial sums are fp32 as well; only the filter gradients need scratch
    assert lib.ddf_hip_backward_workspace_bytes(64, 256, 14, 14, 3, 1, 1, 0, 0, 7, 0) == 8 * n_sf * 4
    assert lib.ddf_hip_backward_workspace_bytes(64, 256, 14, 14, 3, 1, 1, 0, 1, 1, 0) == 0
    # the generic kernels need none, whatever the shape
    assert lib.ddf_hip_backward_workspace_bytes(64, 256, 14, 14, 3, 1, 1, 0, 1, 7, 1) == 0
    assert lib.ddf_hip_backward_workspace_bytes(2, 3, 9, 9, 7, 1, 1, 0, 2, 7, 0) == 0


def test_filter_norm_argument_validation_needs_no_gpu():
    lib = _lib.lib()
    assert lib.ddf_hip_filter_norm(None, None, -1, 1, 9, 4, 1.0, None, None, 1, None) == 1
    assert lib.ddf_hip_filter_norm(None, None, 1, 1, 9, 4, 1.0, None, None, 7, None) == 1
    assert lib.ddf_hip_filter_norm(None, None, 0, 1, 9, 4, 1.0, None, None, 1, None) == 0
    assert lib.ddf_hip_filter_norm(None, None, 2, 1, 9, 4, 1.0, None, None, 1, None) == 1
    assert b'null' in lib.ddf_hip_last_error()


def test_filter_norm_backward_argument_validation_needs_no_gpu():
    lib = _lib.lib()
    bwd = lib.ddf_hip_filter_norm_backward
    assert bwd(None, None, None, None, 1, -1, 9, 4, 1.0, None, 1, None) == 1
    assert bwd(None, None, None, None, 1, 1, 9, 4, 1.0, None, 3, None) == 1
    assert bwd(None, None, None, None, 1, 1, 0, 4, 1.0, None, 1, None) == 0
    assert bwd(None, None, None, None, 2, 1, 9, 4, 1.0, None, 1, None) == 1
    assert b'null' in lib.ddf_hip_last_error()


def test_up_forward_argument_validation_needs_no_gpu():
    import ctypes
    lib = _lib.lib()
    none = (ctypes.c_void_p * 16)()
    up = lib.ddf_hip_up_forward
    assert up(None, none, none, None, 1, 1, 4, 4, 3, 1, 1, 0, 1, None) == 1     # scale 1
    assert b'scale' in lib.ddf_hip_last_error()
    assert up(None, none, none, None, 1, 1, 4, 4, 3, 1, 5, 0, 1, None) == 1     # 25 branches
    assert up(None, none, none, None, 1, 1, 4, 4, 2, 1, 2, 0, 1, None) == 1     # even k
    assert up(None, none, none, None, 1, 1, 4, 4, 7, 1, 2, 0, 1, None) == 2     # no fused kernel
    assert up(None, none, none, None, 0, 8, 4, 4, 3, 1, 2, 0, 1, None) == 0     # empty
    assert up(None, none, none, None, 1, 1, 4, 4, 3, 1, 2, 0, 1, None) == 1
    assert b'null' in lib.ddf_hip_last_error()
    assert _lib.up_forward_covers(3, 2) and not _lib.up_forward_covers(7, 2)


def test_up_backward_validation_and_workspace_need_no_gpu():
    import ctypes
    lib = _lib.lib()
    none = (ctypes.c_void_p * 16)()
    bwd, size = lib.ddf_hip_up_backward, lib.ddf_hip_up_backward_workspace_bytes
    args = (1, 1, 4, 4, 3, 1)
    assert bwd(None, None, none, none, None, none, none, None, 0, *args, 1, 0, 1, 7, None) == 1
    assert b'scale' in lib.ddf_hip_last_error()
    assert bwd(None, None, none, none, None, none, none, None, 0, *args, 2, 0, 1, 0, None) == 0
    assert bwd(None, None, none, none, None, none, none, None, 0, *args, 2, 0, 1, 7, None) == 1
    assert b'null' in lib.ddf_hip_last_error()
    # Lattices and per-branch dX of 4 branches, each padded to 256 bytes; then
    # either the workspace of one 3x3 stride-1 branch (none at this size), or, for
    # all branches as one batch of 8 samples: the filters and the filter gradients
    # of the 4 branches back to back plus that batch's own workspace.
    n_x = 2 * 8 * 6 * 6 * 4
    pad = lambda v: (v + 255) // 256 * 256
    branch = lib.ddf_hip_backward_workspace_bytes(2, 8, 6, 6, 3, 1, 1, 0, 1, 7, 0)
    batch = lib.ddf_hip_backward_workspace_bytes(8, 8, 6, 6, 3, 1, 1, 0, 1, 7, 0)
    n_cf, n_sf = 2 * 8 * 9 * 4, 2 * 9 * 6 * 6 * 4
    staged = 2 * (pad(4 * n_cf) + pad(4 * n_sf))
    assert size(2, 8, 6, 6, 3, 1, 2, 0, 1, 7) == 2 * pad(4 * n_x) + max(pad(branch), staged + pad(batch))
    # fp64 has no batched route
    assert size(2, 8, 6, 6, 3, 1, 2, 0, 2, 7) == 2 * pad(8 * n_x) + pad(
        lib.ddf_hip_backward_workspace_bytes(2, 8, 6, 6, 3, 1, 1, 0, 2, 7, 0))
    # filter gradients only: no dX parts
    assert size(2, 8, 6, 6, 3, 1, 2, 0, 1, 6) == pad(4 * n_x) + max(
        pad(lib.ddf_hip_backward_workspace_bytes(2, 8, 6, 6, 3, 1, 1, 0, 1, 6, 0)),
        staged + pad(lib.ddf_hip_backward_workspace_bytes(8, 8, 6, 6, 3, 1, 1, 0, 1, 6, 0)))
    assert size(2, 8, 6, 6, 3, 1, 1, 0, 1, 7) == 0


def _load_bench():
    import importlib.util
    spec = importlib.util.spec_from_file_location('ddf_bench', os.path.join(ROOT, 'bench.py'))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_bench_algorithmic_bytes_match_the_measurement_plan():
    """Bytes per call with every tensor touched once, at the stage-3 shape:
    forward 26 731 520, backward 40 617 984."""
    bench = _load_bench()
    ab = bench.algorithmic_bytes(64, 256, 14, 14, 3, 1, 4)
    assert ab['fwd'] == 26731520 and ab['bwd'] == 40617984
    assert ab['dx'] + ab['dfilters'] > ab['bwd']   # two calls read dO, CF and SF twice
    half = bench.algorithmic_bytes(64, 64, 56, 56, 3, 1, 2)
    assert half['fwd'] == 55066624 and half['bwd'] == 84443136
    s2 = bench.algorithmic_bytes(32, 128, 56, 56, 3, 2, 4)
    assert s2['fwd'] == 65275904 and s2['bwd'] == 117706752


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    proc = subprocess.run([sys.executable, os.path.join(ROOT, 'bench.py'), '--gpus', '2'],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 2
    assert 'one GPU' in proc.stderr and proc.stdout.strip() == ''


def test_extension_built_after_import_is_picked_up(tmp_path):
    """A process that imports the package before the torch extension exists (a
    clean checkout calling build()) finds it once it has been built: the lookup
    happens at use, a miss is remembered until asked to look again."""
    import glob
    import shutil
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(ddfnet_amd.__file__))
    built = glob.glob(os.path.join(here, '_C*.so'))
    if not built or not _lib.is_built():
        pytest.skip('library or torch extension not built')
    pkg = tmp_path / 'ddfnet_amd'
    pkg.mkdir()
    for path in glob.glob(os.path.join(here, '*.py')):
        shutil.copy(path, pkg)
    script = (
        'import shutil, sys\n'
        'import ddfnet_amd\n'
        'from ddfnet_amd import functional\n'
        'assert functional.extension() is None\n'
        'for path in sys.argv[1:]:\n'
        '    shutil.copy(path, %r)\n'
        'assert functional.extension() is None\n'
        'ext = functional.extension(retry=True)\n'
        'assert ext is not None and hasattr(ext, "ddf")\n' % str(pkg))
    env = dict(os.environ, PYTHONPATH=str(tmp_path))
    subprocess.run([sys.executable, '-c', script, _lib.LIB_PATH] + built, check=True, env=env,
                   cwd=str(tmp_path))
