"""The ROCm backend's host cores run on the CPU against a mock of the C ABI.

`completion.cpp` (stream + completion thread), `signal.cpp` (event / fence state)
and `residency.cpp` (which side of a buffer is current) use no MLX types, so
they link with `tests/rocm_backend/mock_abi.cpp` -- host memory, streams as
threads, fake events -- and `tests/rocm_backend/core_test.cpp` drives them:
buffers retained until the kernel is done, more than ten active tasks without a
later commit (mlx/transforms.cpp:25,271-283), signal before / after wait, host
signals, counting fences, and every residency transition.  Built twice: with
AddressSanitizer + UBSan and with ThreadSanitizer.
"""
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
GLUE = ROOT / "mlx_amd" / "rocm_backend"
HERE = ROOT / "tests" / "rocm_backend"
CORES = ["completion.cpp", "signal.cpp", "residency.cpp"]


def _sanitizer_works(flag, tmp_path):
    src = tmp_path / "probe.cpp"
    src.write_text("int main() { return 0; }\n")
    exe = tmp_path / "probe"
    built = subprocess.run(["g++", f"-fsanitize={flag}", str(src), "-o", str(exe)],
                           capture_output=True)
    return built.returncode == 0 and subprocess.run([str(exe)]).returncode == 0


@pytest.mark.skipif(shutil.which("g++") is None, reason="g++ not present")
@pytest.mark.parametrize("sanitize", ["address,undefined", "thread"])
def test_cores_under_sanitizers(sanitize, tmp_path):
    if not _sanitizer_works(sanitize, tmp_path):
        pytest.skip(f"-fsanitize={sanitize} does not build or run here")
    exe = tmp_path / "core_test"
    cmd = [
        "g++", "-std=c++20", "-g", "-O1", f"-fsanitize={sanitize}", "-fno-omit-frame-pointer",
        "-fno-sanitize-recover=all", "-Wall", "-Werror",
        f"-I{ROOT / 'include'}", f"-I{GLUE}", f"-I{HERE}",
        str(HERE / "core_test.cpp"), str(HERE / "mock_abi.cpp"),
        *[str(GLUE / c) for c in CORES], "-o", str(exe), "-pthread",
    ]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    env = {"ASAN_OPTIONS": "detect_leaks=1", "TSAN_OPTIONS": "halt_on_error=1",
           "UBSAN_OPTIONS": "halt_on_error=1"}
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "all tests passed" in run.stdout
    assert "Sanitizer" not in run.stderr, run.stderr


def test_cores_use_no_mlx_headers():
    for name in CORES + ["completion.h", "signal.h", "residency.h"]:
        text = (GLUE / name).read_text()
        assert '#include "mlx/' not in text, name
