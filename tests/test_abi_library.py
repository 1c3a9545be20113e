"""The C-ABI library loads without a GPU and exports every entry point the headers declare."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pipelink_amd", "libplk_hip.so")


def _declared():
    names = set()
    for header in ("plk_hip.h", "plk_mok.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(plk_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is missing: run __graft_entry__.build()")
    return ctypes.CDLL(LIB)


def test_every_declared_symbol_is_exported(lib):
    declared = _declared()
    assert len(declared) >= 25
    missing = [n for n in declared if not hasattr(lib, n)]
    assert not missing, missing


def test_every_provider_entry_point_is_exported(lib):
    """include/plk_host_abi_v2.h declares abi / query / build / release once per owner suffix."""
    text = open(os.path.join(ROOT, "include", "plk_host_abi_v2.h")).read()
    suffixes = re.findall(r"^PLK_DECLARE_OWNER\((\w+)\)", text, flags=re.M)
    assert suffixes == ["mok_gemm", "mok_act", "mok_framework"]
    missing = [f"pipelink_params_{verb}_{s}" for s in suffixes for verb in ("abi", "query", "build", "release")
               if not hasattr(lib, f"pipelink_params_{verb}_{s}")]
    assert not missing, missing


def test_python_binding_covers_the_headers():
    from pipelink_amd.host.backend import SIGNATURES, load_library

    assert sorted(SIGNATURES) == _declared()
    load_library()


def test_struct_sizes_match_the_c_side():
    """The ctypes mirrors must have the sizes the library checks in struct_bytes."""
    from pipelink_amd.host.backend import DeviceInfo, MokLinkInfo, MokProblem

    assert ctypes.sizeof(MokLinkInfo) == 32
    assert ctypes.sizeof(MokProblem) == 10 * 4 + 2 * 4 + 13 * 8
    assert ctypes.sizeof(DeviceInfo) == 8 * 4 + 8 + 64


def test_missing_library_fails_loudly(tmp_path):
    from pipelink_amd.host.backend import PlkError, load_library

    with pytest.raises(PlkError):
        load_library(str(tmp_path / "nope.so"))
