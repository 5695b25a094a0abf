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

SOURCES = ["rt_api.hip", "rt_kernels.hip", "rt_attn_prefill.hip", "rt_gemv.hip", "rt_mega.hip", "rt_gemm.hip", "rt_llama.hip", "rt_synth.cpp"]

# -packed-fp32-ops off: v_pk_*_f32 forms are kept out of the generated code on purpose.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-munsafe-fp-atomics",  # f32 atomic adds of the split-k GEMM epilogue as hardware atomics (device memory only)
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


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if out:
        sys.stderr.write(out + "\n")


def build_all(verbose: bool = True) -> Path:
    hipcc = find_hipcc()
    OBJ.mkdir(exist_ok=True)
    objs = []

    def compile_one(name: str) -> Path:
        src = CSRC / name
        obj = OBJ / (Path(name).stem + ".o")
        cmd = [hipcc] + HIP_FLAGS + (["-x", "hip"] if name.endswith(".cpp") else []) + ["-c", str(src), "-o", str(obj)]
        if verbose:
            print("[build]", " ".join(cmd), flush=True)
        _run(cmd)
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
