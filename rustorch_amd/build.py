"""Build librustorch_hip for gfx950 with hipcc.

The command lines here are the ones a `build.rs` for a `hip` cargo feature would
run: compile every translation unit with `hipcc --offload-arch=gfx950`, archive
them into `librustorch_hip.a` (what rustc links statically) and also link
`librustorch_hip.so` (what the Python harness loads through ctypes).

Run as `python -m rustorch_amd.build`.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = PKG / "build"
LIB_SO = PKG / "librustorch_hip.so"
LIB_A = PKG / "librustorch_hip.a"

SOURCES = ["rt_api.hip", "rt_kernels.hip", "rt_attn_prefill.hip", "rt_gemv.hip", "rt_gemv_mb.hip", "rt_gemm.hip", "rt_hgemm.hip", "rt_llama.hip", "rt_synth.cpp"]

# -packed-fp32-ops off: v_pk_*_f32 forms are kept out of the generated code on purpose.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-munsafe-fp-atomics",  # the GEMV's in-place residual add (y += row sum) as a returnless hardware f32 atomic (device memory only)
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def find_hipcc() -> str:
    for env in ("HIPCC", ):
        if os.environ.get(env):
            return os.environ[env]
    for root in (os.environ.get("HIP_PATH"), os.environ.get("ROCM_PATH"), "/opt/rocm"):
        if root and (Path(root) / "bin" / "hipcc").exists():
            return str(Path(root) / "bin" / "hipcc")
    found = shutil.which("hipcc")
    if not found:
        raise RuntimeError("hipcc not found (set HIPCC, HIP_PATH or ROCM_PATH)")
    return found


# Kernels whose speed depends on running without private (scratch) memory: the build fails if the compiler gave
# one of them a scratch frame (register spills or an array it could not keep in registers).  One spilling variant
# inside such a kernel slows every launch of it, also the ones that never reach the variant.
NO_SCRATCH = {"rt_gemv.hip": ("qgemv_kernel", "qgemv_lean_kernel"), "rt_gemm.hip": ("qgemm_kernel",), "rt_attn_prefill.hip": ("attn_causal_kernel",),
              "rt_hgemm.hip": ("hgemm_kernel",), "rt_gemv_mb.hip": ("qgemv_mb_q4k_kernel", "qgemv_mb_q6k_kernel"),
              "rt_kernels.hip": ("attn_decode_kernel", "attn_split_kernel", "attn_rows_kernel", "matmul_f32_mfma_kernel")}
RESOURCE_FLAG = "-Rpass-analysis=kernel-resource-usage"


def _run(cmd: list[str]) -> str:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    quiet = ("packed-fp32-ops", RESOURCE_FLAG)
    keep, skip = [], 0
    for l in proc.stdout.splitlines():
        if skip:                         # the source line and caret that follow a remark
            skip -= 1
            continue
        if "remark: Function Name" in l:
            skip = 2
        if l.strip() and not any(q in l for q in quiet):
            keep.append(l)
    if keep:
        sys.stderr.write("\n".join(keep) + "\n")
    return proc.stdout


def check_no_scratch(name: str, log: str) -> None:
    """Parse the compiler's per-kernel resource remarks of one source file."""
    wanted = NO_SCRATCH.get(name, ())
    current = None
    seen = set()
    for l in log.splitlines():
        if "remark: Function Name:" in l:
            current = l.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in l and current:
            size = int(l.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            for k in wanted:
                if k in current:
                    seen.add(k)
                    if size != 0:
                        raise RuntimeError("%s: kernel %s uses %d bytes of scratch per lane (register spills); "
                                           "every launch of it would slow down" % (name, current, size))
    missing = set(wanted) - seen
    if missing:
        raise RuntimeError("%s: no resource report for %s" % (name, ", ".join(sorted(missing))))


def build_all(verbose: bool = True) -> Path:
    hipcc = find_hipcc()
    OBJ.mkdir(exist_ok=True)
    objs = []

    def compile_one(name: str) -> Path:
        src = CSRC / name
        obj = OBJ / (Path(name).stem + ".o")
        extra = [RESOURCE_FLAG] if name in NO_SCRATCH else []
        cmd = [hipcc] + HIP_FLAGS + extra + (["-x", "hip"] if name.endswith(".cpp") else []) + ["-c", str(src), "-o", str(obj)]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        log = _run(cmd)
        if name in NO_SCRATCH:
            check_no_scratch(name, log)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    if LIB_A.exists():
        LIB_A.unlink()
    _run(["ar", "rcs", str(LIB_A)] + [str(o) for o in objs])
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_SO)] + [str(o) for o in objs])
    if verbose:
        print("[build] wrote", LIB_SO, "and", LIB_A, flush=True)
    return LIB_SO


if __name__ == "__main__":
    build_all()
