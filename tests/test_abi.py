"""The C-ABI library loads and exports every function include/*.h declares; failures come back as error codes with
text, never as exceptions or aborts (CPU only: no compute call is made)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(sdx?_[a-z0-9_]+)\s*\(", text)


@pytest.fixture(scope="module")
def library():
    from straydog_amd import abi
    if not os.path.exists(abi.LIBRARY):
        from straydog_amd import build
        build.build()
    return abi.load()


def test_every_declared_function_is_exported_and_typed(library):
    from straydog_amd import abi
    names = set(_declared("straydog_gpu.h")) | set(_declared("straydog_gpu_ext.h"))
    assert len(names) > 35
    assert names == set(abi.SIGNATURES), names ^ set(abi.SIGNATURES)
    for name in names:
        assert getattr(library, name) is not None


def test_failures_are_codes_with_text(library):
    # no GPU here (and on the GPU box an out-of-range ordinal): a null handle and the reason in sd_error()
    handle = library.sd_create(12345, 1 << 20)
    assert handle is None
    assert library.sd_error().decode() != ""
    assert library.sd_buffer(None, 64) is None
    assert b"null" in library.sd_error()
    assert library.sd_op_top_k(None, None, 1, 1, 1, None) == -1
    assert library.sdx_synchronize(None) == -1
    library.sd_destroy(None)   # a no-op


def _golden_symbols():
    """name -> (kind of result, 'real' | 'stub') for every function the reference's gpu/straydog_gpu.h declares."""
    table = {}
    for line in open(os.path.join(ROOT, "tests", "golden", "abi_symbols.txt")):
        if line.strip() and not line.startswith("#"):
            name, kind, state = line.split()
            table[name] = (kind, state)
    return table


def _defined(path):
    import subprocess
    listing = subprocess.run(["nm", "--defined-only", "-g", path], check=True, capture_output=True, text=True).stdout
    return {parts[-1] for parts in (line.split() for line in listing.splitlines()) if len(parts) >= 3 and parts[-2] == "T" and parts[-1].startswith("sd_")}


@pytest.mark.parametrize("artifact", ["libstraydog_gpu.a", "libstraydog_gpu.so"])
def test_library_defines_the_whole_reference_abi(library, artifact):
    # the reference's host links the static archive and binds every declared function (crates/straydog-gpu/build.rs:52):
    # the archive must define each of the 321, no more and no fewer
    golden = _golden_symbols()
    assert len(golden) == 321
    assert _defined(os.path.join(ROOT, "straydog_amd", artifact)) == set(golden)
    assert {name for name, (_, state) in golden.items() if state == "real"} == set(_declared("straydog_gpu.h"))


def test_symbol_list_matches_the_reference_header():
    header = "/root/reference/gpu/straydog_gpu.h"
    if not os.path.exists(header):
        pytest.skip("no reference checkout on this machine; tests/golden/abi_symbols.txt was generated from it")
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_stubs", os.path.join(ROOT, "straydog_amd", "csrc", "gen_stubs.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    golden = _golden_symbols()
    assert [(name, kind) for name, kind in module.declarations(header)] == [(name, kind) for name, (kind, _) in golden.items()]


def test_stubs_fail_cleanly(library):
    golden = _golden_symbols()
    results = {"INT": (ctypes.c_int, -1), "PTR": (ctypes.c_void_p, None), "U64": (ctypes.c_uint64, 0), "I64": (ctypes.c_int64, -1),
               "U32": (ctypes.c_uint32, 0), "VOID": (None, None)}
    stubs = [(name, kind) for name, (kind, state) in golden.items() if state == "stub"]
    assert len(stubs) > 250
    for name, kind in stubs:
        function = getattr(library, name)
        if kind == "STR":
            continue            # (text results: test_text_results_are_never_null)
        function.restype, expected = results[kind]
        function.argtypes = None
        # arguments are ignored (the caller owns them in the C calling convention): pass a few, as a bound caller would
        assert function(None, None, ctypes.c_uint64(3), None) == expected, name
        assert library.sd_error().decode() == f"{name} is not implemented in the attention library"


def test_text_results_are_never_null(library):
    # the host reads a text result without a null check (CStr::from_ptr(ffi::sd_cpu_error()) after any failed CPU-engine call,
    # crates/straydog-engine/src/gpu.rs:3831-3838): every function that answers text answers some, and sd_cpu_error the reason
    # of the thread's last refusal
    golden = _golden_symbols()
    texts = [name for name, (kind, _) in golden.items() if kind == "STR"]
    assert set(texts) == {"sd_error", "sd_cpu_error", "sd_cpu_experts_isa"}
    for name in texts:
        function = getattr(library, name)
        function.restype, function.argtypes = ctypes.c_char_p, None
    library.sd_cpu_experts_create.restype, library.sd_cpu_experts_create.argtypes = ctypes.c_void_p, None
    assert library.sd_cpu_experts_create(ctypes.c_uint32(4), ctypes.c_uint32(0)) is None
    assert library.sd_cpu_error() == b"sd_cpu_experts_create is not implemented in the attention library"
    assert library.sd_cpu_error() == library.sd_error()
    isa = library.sd_cpu_experts_isa(None)
    assert isa is not None and b"sd_cpu_experts_isa is not implemented" in isa
    assert library.sd_error() is not None


def test_backend_refuses_a_missing_library(tmp_path):
    from straydog_amd import abi
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        abi.load(str(tmp_path / "absent.so"))
