"""What the compiler made of the decode GEMV kernels, read from the assembly it writes for gfx950 (no GPU needed: hipcc
cross-compiles).  Three properties that cost speed silently when lost, none of which a numerical test can see:

  * no waterfall loop around a weight load -- the per-row buffer descriptors stay wave-uniform, in scalar registers (a
    descriptor the compiler cannot prove uniform is served one distinct value at a time, in a loop over the lanes);
  * the steady-state loops of the lean kernels wait for their loads one by one (`s_waitcnt vmcnt(n)`, n > 0) and never
    for everything (`vmcnt(0)`), which would include the prefetch issued a moment before;
  * every weight load in those loops is a buffer load (range-checked window), none a plain global load.
"""
import re
import subprocess

import pytest

from rustorch_amd import build as rt_build


@pytest.fixture(scope="module")
def gemv_asm(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa") / "rt_gemv.s"
    src = rt_build.CSRC / "rt_gemv.hip"
    try:
        hipcc = rt_build.find_hipcc()
    except RuntimeError as e:
        pytest.skip(str(e))
    cmd = [hipcc] + rt_build.HIP_FLAGS + ["-I", str(rt_build.CSRC), "-I", str(rt_build.PKG.parent / "include"),
                                                         "--cuda-device-only", "-S", str(src), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
    return out.read_text().split("\n")


def kernels(lines):
    """name -> (instructions, label -> index of the instruction that follows it)"""
    out, cur = {}, None
    for l in lines:
        m = re.match(r"^(_ZN2rt\S+):", l)
        if m:
            cur = m.group(1)
            out[cur] = ([], {})
            continue
        if cur is None:
            continue
        t = l.strip()
        ins, labels = out[cur]
        m = re.match(r"^(\.LBB\d+_\d+):", t)
        if m:
            labels[m.group(1)] = len(ins)
        elif t and not t.startswith((";", ".")):
            ins.append(t.split(";")[0].strip())
        if "s_endpgm" in l:
            cur = None
    return out


def loops(ins, labels):
    """(first, last) instruction index of every backward branch's range"""
    for i, t in enumerate(ins):
        m = re.match(r"^s_(?:cbranch_\w+|branch)\s+(\.LBB\d+_\d+)", t)
        if m and m.group(1) in labels and labels[m.group(1)] <= i:
            yield labels[m.group(1)], i


def test_weight_descriptors_stay_scalar(gemv_asm):
    ks = kernels(gemv_asm)
    names = [k for k in ks if "qgemv_kernel" in k or "qgemv_lean_kernel" in k]
    assert len(names) >= 7, names
    for name in names:
        ins, labels = ks[name]
        assert sum(t.startswith("buffer_load") for t in ins) > 50, name
        for a, b in loops(ins, labels):
            body = ins[a:b + 1]
            # a waterfall loop: short, ends on "any lanes left", reads one lane's value and holds a load
            if len(body) < 60 and ins[b].startswith("s_cbranch_execnz") and any("v_readfirstlane" in t for t in body):
                assert not any(t.startswith("buffer_load") for t in body), "%s: waterfall loop around a buffer load:\n%s" % (name, "\n".join(body))


def test_lean_steady_state_waits_per_load(gemv_asm):
    ks = kernels(gemv_asm)
    names = [k for k in ks if "qgemv_lean_kernel" in k]
    assert len(names) == 5, names
    for name in names:
        ins, labels = ks[name]
        found = 0
        all_loops = list(loops(ins, labels))
        for a, b in all_loops:
            body = ins[a:b + 1]
            n_dot = sum(t.startswith("v_dot4") for t in body)
            n_load = sum(t.startswith("buffer_load") for t in body)
            # the two-step steady-state loops: two requests' worth of weight loads and their dot products, no loop inside
            # but the lane scan of a returnless atomic
            if n_dot < 32 or n_load < 4 or any(o != (a, b) and a <= o[0] and o[1] <= b and sum(t.startswith("v_dot4") for t in ins[o[0]:o[1] + 1]) >= 16 for o in all_loops):
                continue
            found += 1
            assert not any(t.startswith("global_load") for t in body), "%s: a plain global load in a steady-state loop" % name
            waits = [int(re.search(r"vmcnt\((\d+)\)", t).group(1)) for t in body if t.startswith("s_waitcnt") and "vmcnt" in t]
            assert waits and min(waits) > 0, "%s: loop of %d instructions waits vmcnt%s" % (name, len(body), waits)
        assert found >= 6, (name, found)
