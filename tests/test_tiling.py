"""Host logic of the launch plans (GEMMs: 2D XCD regions, panels, K split of tail tiles; bandwidth-bound kernels: K
slices x column tiles): a small host program enumerates every workgroup of many launches and checks that each output
tile, and each K range or slice of it, is computed exactly once."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_tile_exactly_once(tmp_path):
    hipcc = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
    if not os.path.exists(hipcc):
        pytest.skip('hipcc not available')
    exe = str(tmp_path / 'tiling_check')
    cmd = [hipcc, '--offload-arch=gfx950', '-O1', '-std=c++17', '-I', os.path.join(ROOT, 'hidet_amd', 'csrc'), '-I',
           os.path.join(ROOT, 'include'), os.path.join(ROOT, 'tests', 'host', 'tiling_check.hip'), '-o', exe]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.startswith('ok'), r.stdout[-2000:]
