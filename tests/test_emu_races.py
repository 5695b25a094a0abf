"""The emulation's race detector checks itself: tests/emu/emu_race_selftest.cpp is built under ThreadSanitizer with and
without a missing workgroup barrier; the first build has to be reported as a data race, the second has to run clean.
(The library's own kernels run under the same detector through `python tests/emu/build_emulated.py OUT --races --pytest ...`.)"""
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT / "tests" / "emu"))
import build_emulated  # noqa: E402


@pytest.mark.skipif(not Path(build_emulated.CLANG).exists(), reason="needs ROCm's clang++")
@pytest.mark.parametrize("racy", [False, True])
def test_missing_barrier_between_waves_is_reported(tmp_path, racy):
    exe = tmp_path / "selftest"
    # one translation unit: the kernel is compiled with the instrumentation, the scheduler (emu_fibers.h) marks itself out
    cmd = [build_emulated.CLANG, "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-mllvm", "-tsan-instrument-func-entry-exit=0", "-DEMU_TSAN=1",
           "-I", str(ROOT / "tests" / "emu"), str(ROOT / "tests" / "emu" / "emu_race_selftest.cpp"), "-o", str(exe)]
    if racy:
        cmd.insert(1, "-DRACY=1")
    subprocess.run(cmd, check=True)
    r = subprocess.run([str(exe)], env=dict(os.environ, TSAN_OPTIONS="halt_on_error=0:exitcode=66"), capture_output=True, text=True, timeout=300)
    assert "ran sum" in r.stdout, r.stdout + r.stderr
    if racy:
        assert r.returncode == 66 and "data race" in r.stderr and "kernel" in r.stderr, r.stderr[-3000:]
    else:
        assert r.returncode == 0 and "ThreadSanitizer" not in r.stderr, r.stderr[-3000:]
