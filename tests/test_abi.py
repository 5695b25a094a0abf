"""The C-ABI library loads without a GPU and exports exactly what include/rustorch_hip.h declares."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "rustorch_hip.h"


def header_symbols():
    text = HEADER.read_text()
    return re.findall(r"RT_HIP_API\s+[\w\s\*]+?\b(rt_\w+)\s*\(", text)


def test_header_symbols_are_exported_and_bound(lib):
    from rustorch_amd import _lib
    syms = header_symbols()
    assert len(syms) >= 40 and len(set(syms)) == len(syms)
    for s in syms:
        assert hasattr(lib, s), "missing export %s" % s
    assert sorted(syms) == sorted(_lib.SIGNATURES), "ctypes table and header disagree"


def test_rust_binding_in_the_integration_notes_is_generated_from_the_header():
    """The integration notes hold the Rust `extern "C"` module a maintainer would add; it is generated from the header, declares
    every exported function with the header's argument count, pointer-ness and return kind, and agrees with the ctypes table."""
    import ctypes as C
    from rustorch_amd import _lib, ffi_gen
    assert ffi_gen.doc_block() == ffi_gen.generate(), "run python -m rustorch_amd.ffi_gen --write"
    block = ffi_gen.doc_block()
    decls = dict(re.findall(r"^    pub fn (rt_\w+)\((.*)\) -> [^;]+;$", block, flags=re.M))
    rets = dict(re.findall(r"^    pub fn (rt_\w+)\(.*\) -> ([^;]+);$", block, flags=re.M))
    stubs = set(re.findall(r"^    pub unsafe fn (rt_\w+)\(", block, flags=re.M))
    assert sorted(decls) == sorted(header_symbols()) and stubs == set(decls)
    for name, (res, args) in _lib.SIGNATURES.items():
        rust_args = [a.split(": ", 1)[1] for a in decls[name].split(", ")] if decls[name] else []
        assert len(rust_args) == len(args), name
        for ra, ca in zip(rust_args, args):
            is_ptr = ra.startswith("*")
            c_ptr = ca in (C.c_void_p, C.c_char_p) or hasattr(ca, "contents")
            assert is_ptr == c_ptr, "%s: %s against %s" % (name, ra, ca)
            if not is_ptr:
                want = {C.c_int: ("i32",), C.c_float: ("f32",)}.get(ca, ("usize", "u64"))       # size_t and uint64_t are one ctypes class here
                assert ra in want, "%s: %s against %s" % (name, ra, ca)
        assert rets[name] == {C.c_int: "i32", C.c_size_t: "usize", C.c_char_p: "*const std::os::raw::c_char"}[res], name


def test_static_archive_holds_the_same_entry_points(lib):
    import subprocess
    a = ROOT / "rustorch_amd" / "librustorch_hip.a"
    if not a.exists():
        pytest.skip("static archive not built")
    out = subprocess.run(["nm", "-g", "--defined-only", str(a)], stdout=subprocess.PIPE, text=True).stdout
    defined = set(re.findall(r"\bT (rt_\w+)", out))
    assert set(header_symbols()) <= defined


def test_type_table_matches_reference_type_size(lib):
    # example-cli/src/model/formats/gguf.rs:78-99,125-144
    from rustorch_amd import GGMLType
    for t, size, elems in ((0, 4, 1), (1, 2, 1), (2, 18, 32), (3, 20, 32), (6, 22, 32), (7, 24, 32), (8, 34, 32), (9, 36, 32), (10, 84, 256), (11, 110, 256), (12, 144, 256), (13, 176, 256),
                           (14, 210, 256)):
        assert lib.rt_hip_type_block_bytes(t) == size and lib.rt_hip_type_block_elems(t) == elems
        assert GGMLType(t).type_size() == size and GGMLType(t).block_elems() == elems
    assert lib.rt_hip_type_block_bytes(15) == 0 and lib.rt_hip_type_block_bytes(99) == 0  # no kernel (Q8_K): reported, not guessed
    # the reference's own unit tests: ids 0,1,2 and the unknown-id error (gguf.rs:414-426)
    assert GGMLType.from_u32(0) is GGMLType.F32 and GGMLType.from_u32(1) is GGMLType.F16 and GGMLType.from_u32(2) is GGMLType.Q4_0
    with pytest.raises(ValueError, match="Unknown GGML type"):
        GGMLType.from_u32(999)
    assert (GGMLType.F32.type_size(), GGMLType.F16.type_size(), GGMLType.I8.type_size()) == (4, 2, 1)
    assert GGMLType.Q4_K.row_bytes(4096) == 2304 and GGMLType.Q6_K.row_bytes(11008) == 9030
    with pytest.raises(ValueError):
        GGMLType.Q4_K.row_bytes(1000)


def test_null_and_missing_device_are_errors_not_crashes(lib):
    from rustorch_amd import _lib, DeviceNotAvailable, InvalidParameters
    from rustorch_amd.executor import HipKernelExecutor, device_count
    assert lib.rt_hip_create(0, None) == 1
    assert lib.rt_hip_synchronize(None) == 1
    assert lib.rt_hip_destroy(None) == 0 and lib.rt_hip_qweight_free(None, None) == 0
    ctx = C.c_void_p()
    assert lib.rt_hip_create(4096, C.byref(ctx)) == 3 and not ctx.value
    assert b"hip:4096" in lib.rt_hip_last_error(None)
    with pytest.raises(DeviceNotAvailable):
        HipKernelExecutor(4096)
    with pytest.raises(InvalidParameters):
        _lib.check(lib.rt_hip_malloc(None, 16, None))
    if device_count() == 0:
        with pytest.raises(DeviceNotAvailable):   # no silent CPU fallback
            HipKernelExecutor(0)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from rustorch_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.load()
