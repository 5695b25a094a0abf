"""The decode GEMV's device code -- the general path and the lean path of the benchmark's formats -- compiled as host
C++ and run as fibers under AddressSanitizer (tests/emu/emu_gemv.cpp) on the grids the launcher's planner lays out:
no access outside the buffers a launch is handed (short rows, ragged last passes, more waves than rows, the gate / up
pair form, in-place residuals, all three staging modes), the two paths bit-identical, both within the held tolerance
of the oracle's f64 dot products."""
import os
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
CLANG = "/opt/rocm/llvm/bin/clang++"


@pytest.mark.skipif(not (Path(CLANG).exists() and shutil.which("gcc")), reason="needs ROCm's clang++ and gcc")
def test_gemv_device_code_as_cpu_fibers_under_asan(tmp_path):
    obj = tmp_path / "rt_oracle.o"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-fopenmp", "-c", str(ROOT / "oracle" / "rt_oracle.c"), "-o", str(obj)], check=True)
    exe = tmp_path / "emu_gemv"
    subprocess.run([CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=address", "-DRT_EMULATED=1", "-I", str(ROOT / "tests" / "emu"),
                    "-I", str(ROOT / "rustorch_amd" / "csrc"), "-I", str(ROOT / "include"), str(ROOT / "tests" / "emu" / "emu_gemv.cpp"),
                    str(ROOT / "rustorch_amd" / "csrc" / "rt_synth.cpp"), str(obj), "-o", str(exe), "-fopenmp"], check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    r = subprocess.run([str(exe)], env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "EMU OK" in r.stdout
    assert "ERROR: AddressSanitizer" not in r.stderr
