"""The library's own sources built as host C++ (tests/emu/build_emulated.py: every GPU thread a fiber, device memory as
exact-size heap blocks, AddressSanitizer on) and a selection of the GPU tests run against that build, through the same
C-ABI and the same Python layer.  What it adds to the GPU run: an access outside a buffer, a barrier that not every
thread reaches or a host-side sizing mistake stops this run with a report; on the device it would be a fault.  What it
does not show: timing, and anything that depends on how the hardware interleaves waves.

The selection keeps to sizes a CPU finishes in a few minutes; `python tests/emu/build_emulated.py OUT_DIR --pytest ...`
runs any other GPU test the same way."""
import os
import shutil
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT / "tests" / "emu"))
import build_emulated  # noqa: E402

SELECTION = [
    "tests/test_gpu_ops.py",
    "tests/test_gpu_dequant.py",
    "tests/test_gpu_failures.py",
    "tests/test_qmatmul.py",
    "tests/test_gpu_gemv.py::test_gemv_edge_inputs",
    "tests/test_gpu_gemv.py::test_gemv_config_shapes_batch1_and_8[C3_q]",          # the benchmark's own matrices, whole
    "tests/test_gpu_gemv.py::test_gemv_config_shapes_batch1_and_8[C3_gate]",
    "tests/test_gpu_gemv.py::test_gemv_config_shapes_batch1_and_8[C3_v]",
    "tests/test_gpu_gemv.py::test_gemv_config_shapes_batch1_and_8[C3_down]",
    "tests/test_gpu_gemv.py::test_grouped_launch_equals_single_launches",
    "tests/test_gpu_gemv.py::test_several_weights_against_one_batch",
    "tests/test_gpu_gemv.py::test_device_pointer_form_and_errors",
    "tests/test_gpu_gemv.py::test_dense_matmul_f32_kat",
    "tests/test_gpu_gemv.py::test_dense_matmul_on_resident_buffers_and_batches",
    "tests/test_z_optin_paths.py",                                                  # the lean GEMV and the dense matrix-core kernel, switched on per test
    "tests/test_gpu_gemv.py::test_batches_of_two_to_eight_on_the_matrix_cores[37-256-12]",
    "tests/test_gpu_gemv.py::test_batches_of_two_to_eight_on_the_matrix_cores[16-768-14]",
    "tests/test_gpu_gemv.py::test_batches_of_two_to_eight_on_the_matrix_cores[1-4096-12]",
    "tests/test_gpu_gemv.py::test_batches_of_two_to_eight_on_the_matrix_cores[300-11008-14]",
    "tests/test_gpu_gemm.py::test_single_superblock_odd_counts_and_tiny_matrices",
    "tests/test_gpu_gemm.py::test_other_formats_and_small_m_use_the_row_form",
    "tests/test_gpu_gemm.py::test_three_to_fifteen_rows_go_eight_at_a_time[100-11008-12]",
    "tests/test_gpu_gemm.py::test_three_to_fifteen_rows_go_eight_at_a_time[100-11008-14]",
    "tests/test_gpu_llama.py::test_model_from_gguf_file_equals_direct_upload",
    "tests/test_z_batch_decode.py::test_three_sequences_on_a_small_model",        # several sequences side by side
    "tests/test_z_batch_decode.py::test_batch_arguments_are_checked",
]


@pytest.mark.skipif(not (Path(build_emulated.CLANG).exists() and shutil.which("gcc")), reason="needs ROCm's clang++ and gcc")
def test_gpu_tests_pass_on_the_emulated_library_under_asan(tmp_path):
    so = build_emulated.build(tmp_path / "emulated")
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", *SELECTION, "-m", "gpu", "-x", "-q", "-n", "4", "-p", "no:cacheprovider"],
                       cwd=ROOT, env=build_emulated.environment(so), capture_output=True, text=True, timeout=1500)
    tail = r.stdout[-4000:] + r.stderr[-4000:]
    assert "AddressSanitizer" not in r.stdout + r.stderr, tail
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and "failed" not in r.stdout, tail


# the race detector's share of the same selection: what passes data between waves through LDS
RACE_SELECTION = [
    "tests/test_gpu_ops.py",
    "tests/test_gpu_gemv.py::test_gemv_edge_inputs",
    "tests/test_gpu_gemv.py::test_gemv_config_shapes_batch1_and_8[C3_down]",       # rows of three passes dealt out over the waves
    "tests/test_gpu_gemv.py::test_grouped_launch_equals_single_launches",
    "tests/test_gpu_gemv.py::test_batches_of_two_to_eight_on_the_matrix_cores[300-11008-14]",
    "tests/test_z_optin_paths.py::test_dense_matmul_on_the_matrix_cores",
    "tests/test_z_optin_paths.py::test_lean_gemv_edge_inputs",
    "tests/test_z_optin_paths.py::test_lean_gemv_config_shapes[lean-C3_down]",
    "tests/test_z_optin_paths.py::test_lean_gemv_config_shapes[lean-five-waves-C3_down]",
    "tests/test_gpu_gemm.py::test_single_superblock_odd_counts_and_tiny_matrices",
    "tests/test_gpu_gemm.py::test_three_to_fifteen_rows_go_eight_at_a_time[100-11008-12]",
    "tests/test_z_batch_decode.py::test_three_sequences_on_a_small_model",        # the per-sequence attention folds its groups through LDS
]


@pytest.mark.skipif(not (Path(build_emulated.CLANG).exists() and shutil.which("gcc")), reason="needs ROCm's clang++ and gcc")
def test_gpu_tests_show_no_race_between_waves_on_the_emulated_library(tmp_path):
    """The same sources under ThreadSanitizer with a wave as a thread of the detector (tests/emu/emu_fibers.h): an access of
    one wave to what another wrote, with no workgroup barrier between, ends the run with the detector's exit code."""
    so = build_emulated.build(tmp_path / "emulated", sanitizer="thread")
    # one process, output not captured by pytest: the detector's reports reach stderr and its exit code is the run's
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", *RACE_SELECTION, "-m", "gpu", "-x", "-q", "-s", "-p", "no:cacheprovider"],
                       cwd=ROOT, env=build_emulated.environment(so, "thread"), capture_output=True, text=True, timeout=1500)
    tail = r.stdout[-4000:] + r.stderr[-4000:]
    assert "ThreadSanitizer" not in r.stdout + r.stderr, tail
    assert r.returncode == 0, tail
    assert " passed" in r.stdout and "failed" not in r.stdout, tail
