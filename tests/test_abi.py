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


def test_static_archive_is_built():
    assert os.path.exists(os.path.join(ROOT, "straydog_amd", "libstraydog_gpu.a"))


def test_backend_refuses_a_missing_library(tmp_path):
    from straydog_amd import abi
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        abi.load(str(tmp_path / "absent.so"))
