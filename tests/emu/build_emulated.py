"""Builds the library's own sources as host C++ against the stand-in HIP headers of tests/emu: every GPU thread a fiber,
every device allocation an exact-size heap block under AddressSanitizer (with the undefined-behaviour sanitizer's checks of
alignment, array bounds, shifts, signed overflow and conversions beside it: any of them stops the run).  TEST INFRASTRUCTURE: the result is loaded by
tests only (RUSTORCH_HIP_LIBRARY names it), to run the same tests that run on the GPU -- at small sizes -- where an access
outside a buffer stops the run with a report instead of faulting a device.

The one thing host C++ cannot read is the launch syntax, so the sources are copied with every
`kernel<<<grid, block, lds, stream>>>(args)` rewritten as `EMU_LAUNCH((kernel), grid, block, lds, stream, args)`,
every `asm(...)` statement as a call of the stand-in header's interpreter of the few instructions the sources write by
hand, and the attributes only the GPU target knows (LDS address spaces, occupancy hints) dropped; nothing else changes, and lines keep their numbers."""
from __future__ import annotations

import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parents[2]
CSRC = ROOT / "rustorch_amd" / "csrc"
EMU = ROOT / "tests" / "emu"
CLANG = "/opt/rocm/llvm/bin/clang++"
SOURCES = ["rt_api.hip", "rt_kernels.hip", "rt_gemv.hip", "rt_gemv_mb.hip", "rt_gemm.hip", "rt_hgemm.hip", "rt_attn_prefill.hip", "rt_llama.hip", "rt_synth.cpp"]


def _match_back(src: str, end: int) -> int:
    """Start of the kernel expression that ends at `end`: an identifier (with namespaces) and its template arguments."""
    i = end
    while i > 0 and src[i - 1].isspace():
        i -= 1
    if i > 0 and src[i - 1] == ">":
        depth = 0
        while i > 0:
            i -= 1
            if src[i] == ">":
                depth += 1
            elif src[i] == "<":
                depth -= 1
                if depth == 0:
                    break
    while i > 0 and (src[i - 1].isalnum() or src[i - 1] in "_:"):
        i -= 1
    return i


def _match_paren(src: str, start: int) -> int:
    """Index just past the parenthesis that closes the one at `start`."""
    depth = 0
    for i in range(start, len(src)):
        if src[i] == "(":
            depth += 1
        elif src[i] == ")":
            depth -= 1
            if depth == 0:
                return i + 1
    raise ValueError("unbalanced parentheses after a launch")


def rewrite_launches(src: str) -> str:
    out, pos = [], 0
    while True:
        at = src.find("<<<", pos)
        if at < 0:
            break
        close = src.index(">>>", at)
        k0 = _match_back(src, at)
        args0 = close + 3
        while src[args0].isspace():
            args0 += 1
        assert src[args0] == "(", "launch without an argument list near: " + src[at - 40:at + 40]
        args1 = _match_paren(src, args0)
        kernel, config, args = src[k0:at].strip(), src[at + 3:close].strip(), src[args0 + 1:args1 - 1].strip()
        out.append(src[pos:k0])
        out.append("EMU_LAUNCH((%s), %s%s)" % (kernel, config, (", " + args) if args else ""))
        pos = args1
    out.append(src[pos:])
    return "".join(out)


def _split_top(text: str, sep: str) -> list[str]:
    """Split at `sep` outside parentheses and string literals."""
    parts, depth, start, i, in_str = [], 0, 0, 0, False
    while i < len(text):
        c = text[i]
        if in_str:
            if c == "\\":
                i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True
        elif c == "(":
            depth += 1
        elif c == ")":
            depth -= 1
        elif c == sep and depth == 0:
            parts.append(text[start:i])
            start = i + 1
        i += 1
    parts.append(text[start:])
    return parts


def rewrite_asm(src: str) -> str:
    """asm [volatile] ("template" : outputs : inputs : clobbers) -> emu_asm("template", emu_out(o)..., emu_in(i)...)."""
    out, pos = [], 0
    while True:
        m = re.search(r"\basm\s*(volatile\s*)?\(", src[pos:])
        if not m:
            break
        a0 = pos + m.start()
        p0 = pos + m.end() - 1
        p1 = _match_paren(src, p0)
        sections = _split_top(src[p0 + 1:p1 - 1], ":")
        template = sections[0].strip()
        ops = []
        for kind, sec in (("emu_out", sections[1] if len(sections) > 1 else ""), ("emu_in", sections[2] if len(sections) > 2 else "")):
            for item in _split_top(sec, ","):
                item = item.strip()
                if not item:
                    continue
                cm = re.match(r'"([^"]*)"\s*\((.*)\)$', item, re.S)
                assert cm, "operand not understood: " + item
                ops.append("%s(%s)" % ("emu_out" if kind == "emu_out" or cm.group(1).startswith("+") else "emu_in", cm.group(2).strip()))
        out.append(src[pos:a0])
        out.append("emu_asm(%s)" % ", ".join([template] + ops))
        pos = p1
    out.append(src[pos:])
    return "".join(out)


def rewrite_predicated_lds(src: str) -> str:
    """`if (cond) lds_write16<..>(..);` -> the same with `else emu_wave_sync();`.

    On the device a wave issues each of its hand-written LDS instructions (the sources' lds_read* / lds_write* helpers)
    once, for all lanes, some of them masked; the emulation makes every such instruction a rendezvous of the wave's lanes.
    A lane whose predicate is false has to turn up at that rendezvous too, or it pairs up with the others' next one."""
    return re.sub(r"\bif \(([^;{}]*?)\) (lds_(?:read|write)\w*<[^;]*;)", r"if (\1) \2 else emu_wave_sync();", src)


def to_host_cpp(src: str) -> str:
    src = rewrite_predicated_lds(src)
    src = re.sub(r"__attribute__\(\(address_space\(\d\)\)\)", "", src)
    src = re.sub(r"__attribute__\(\(amdgpu_\w+\([^()]*\)\)\)", "", src)       # occupancy hints of kernels
    return rewrite_asm(rewrite_launches(src))


# The two instrumented builds.  "address": out-of-bounds and misaligned accesses, indices outside fixed-size arrays, shifts by
# too much, signed overflow, float-to-int conversions out of range, integer division by zero (each ends the run).  "thread": a wave is a thread of the race
# detector (emu_fibers.h); function entry / exit hooks are off because the 64 lanes of a wave share one detector context
# while each has a call stack of its own.
SANITIZERS = {
    "address": ["-fsanitize=address,alignment,bounds,shift-exponent,signed-integer-overflow,float-cast-overflow,integer-divide-by-zero",
                "-fno-sanitize-recover=all", "-shared-libasan"],
    "thread": ["-fsanitize=thread", "-shared-libsan", "-mllvm", "-tsan-instrument-func-entry-exit=0"],
    "none": [],        # no checks: several times faster, for looking at the numerics of sizes the checked builds take hours over
}


def build(out_dir: Path, verbose: bool = False, sanitizer: str = "address") -> Path:
    out_dir.mkdir(parents=True, exist_ok=True)
    gen = out_dir / "src"
    gen.mkdir(exist_ok=True)
    san = SANITIZERS[sanitizer]
    flags = ["-std=c++17", "-O2", "-g", "-fPIC", *san, "-fno-omit-frame-pointer", "-DRT_EMULATED=1",
             "-Wno-unknown-attributes", "-Wno-unused-value", "-I", str(EMU), "-I", str(CSRC), "-I", str(ROOT / "include")]
    jobs = []
    for name in SOURCES:
        text = to_host_cpp((CSRC / name).read_text())
        cpp = gen / (Path(name).stem + ".cpp")
        cpp.write_text('#line 1 "%s"\n%s' % (CSRC / name, text))
        jobs.append((cpp, out_dir / (Path(name).stem + ".o")))
    jobs.append((EMU / "emu_library.cpp", out_dir / "emu_library.o"))

    def compile_one(job):
        src, obj = job
        mine = list(flags)
        if sanitizer == "thread" and src.name == "emu_library.cpp":
            # the fiber scheduler tells the race detector what it does (EMU_TSAN) but is not itself watched
            mine = [f for f in mine if f not in san] + ["-DEMU_TSAN=1"]
        cmd = [CLANG, *mine, "-x", "c++", "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[emu build]", " ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("emulated build of %s failed:\n%s" % (src.name, r.stderr[-6000:]))

    with ThreadPoolExecutor(max_workers=min(4, os.cpu_count() or 1)) as pool:
        list(pool.map(compile_one, jobs))
    so = out_dir / "librustorch_hip_emulated.so"
    r = subprocess.run([CLANG, "-shared", *[f for f in san if not f.startswith("-mllvm") and not f.startswith("-tsan")], *[str(o) for _, o in jobs], "-o", str(so)],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link of the emulated library failed:\n" + r.stderr[-6000:])
    return so


def sanitizer_runtime(sanitizer: str = "address") -> str:
    if sanitizer == "none":
        return ""
    name = {"address": "asan", "thread": "tsan"}[sanitizer]
    return subprocess.run([CLANG, "-print-file-name=libclang_rt.%s-x86_64.so" % name], capture_output=True, text=True, check=True).stdout.strip()


def environment(so: Path, sanitizer: str = "address") -> dict:
    """The environment of a Python process that is to load the emulated library instead of the GPU one."""
    env = dict(os.environ)
    env["RUSTORCH_HIP_LIBRARY"] = str(so)
    # the sanitizer's runtime has to be in the process before the library is; whatever is preloaded already stays
    env["LD_PRELOAD"] = ":".join(x for x in (sanitizer_runtime(sanitizer), env.get("LD_PRELOAD", "")) if x)
    # a fake stack per fiber (the default's use-after-return check) costs more than the kernels themselves
    env["ASAN_OPTIONS"] = "detect_leaks=0:detect_stack_use_after_return=0:verify_asan_link_order=0"
    # a race is a failure of the run, reported once per place
    env["TSAN_OPTIONS"] = "halt_on_error=0:exitcode=66:report_signal_unsafe=0:history_size=4:suppressions=%s" % (EMU / "tsan.supp")
    env["PYTHONPATH"] = os.pathsep.join(x for x in (str(ROOT), env.get("PYTHONPATH", "")) if x)
    return env


if __name__ == "__main__":
    if len(sys.argv) < 2:
        sys.exit("usage: python tests/emu/build_emulated.py OUT_DIR [--races | --unchecked] [--pytest PYTEST_ARGS... | --run SCRIPT ARGS...]\n"
                 "  --races: the ThreadSanitizer build (a wave is a thread: unordered accesses of two waves are reported)\n"
                 "  --unchecked: no sanitizer (faster; numerics only)\n"
                 "  builds the emulated library into OUT_DIR; with --pytest, then runs `pytest -m gpu PYTEST_ARGS` against it;\n"
                 "  with --run, a Python script (tests/emu/fuzz_shapes.py for one)")
    kind = "thread" if "--races" in sys.argv else ("none" if "--unchecked" in sys.argv else "address")
    for flag in ("--races", "--unchecked"):
        if flag in sys.argv:
            sys.argv.remove(flag)
    lib = build(Path(sys.argv[1]), verbose="--pytest" not in sys.argv and "--run" not in sys.argv, sanitizer=kind)
    print(lib)
    if "--run" in sys.argv:
        args = sys.argv[sys.argv.index("--run") + 1:]
        sys.exit(subprocess.run([sys.executable, "-u", *args], cwd=ROOT, env=environment(lib, kind)).returncode)
    if "--pytest" in sys.argv:
        args = sys.argv[sys.argv.index("--pytest") + 1:]
        sys.exit(subprocess.run([sys.executable, "-u", "-m", "pytest", "-m", "gpu", *args], cwd=ROOT, env=environment(lib, kind)).returncode)
