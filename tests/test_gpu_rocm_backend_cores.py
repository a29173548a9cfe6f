"""The ROCm backend's host cores (completion queue, signal, buffer residency)
run against the real HIP library on the GPU: `tests/rocm_backend/gpu_core_test.cpp`,
built ahead of time by `mlx_amd/_build.py`."""
import os
import subprocess

import pytest

from mlx_amd import _build

pytestmark = pytest.mark.gpu


def test_cores_on_the_gpu():
    exe = _build.GLUE_GPU_TEST
    assert os.path.isfile(exe), f"{exe} is not built: run `python -m mlx_amd._build`"
    run = subprocess.run([exe], capture_output=True, text=True, timeout=150)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all tests passed" in run.stdout
