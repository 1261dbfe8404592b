"""The C-ABI library loads without a GPU and exports every entry point include/crusader_hip.h declares
(no compute calls here)."""
import ctypes
import os
import re

from crusaderbackend_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "crusader_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(crb_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 15
    lib = ctypes.CDLL(capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
        assert n in capi.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(capi.SIGNATURES) == names


def test_abi_version_and_error_string_without_gpu():
    lib = capi.load()
    assert lib.crb_abi_version() >= 1000
    # argument validation happens before any device work, so it can be exercised on a CPU-only host
    assert lib.crb_sgemm_nn(None, None, None, 1, 1, 1, 1, None) == capi.CRB_ENULL
    assert b"null operand" in lib.crb_last_error_string()
    g = capi.ConvGeom.make(1, 1, 4, 4, 1, 3, 3, 1, 1, 0, 0, OH=3, OW=2)
    assert capi.conv_wgrad_workspace_bytes(g) == 0  # invalid geometry -> 0 and an error message
    assert b"relationship did not satisfy" in lib.crb_last_error_string()


def test_conv_geom_layout_matches_header():
    assert ctypes.sizeof(capi.ConvGeom) == 13 * 4
    g = capi.ConvGeom.make(128, 16, 32, 32, 32, 3, 3, 2, 2, 1, 1)
    assert (g.OH, g.OW) == (16, 16)


def test_frozen_call_replays_the_launching_calls_only():
    # null operands fail validation before any device work: the replay must issue the same call and raise the same error
    seen = []

    def wrapper():
        seen.append(capi.gemm_workspace_bytes(64, 64, 64, 1))  # a size query: used by the wrapper, not replayed
        lib = capi.load()
        seen.append(lib.crb_sgemm_nn(None, None, None, 1, 1, 1, 1, None))

    call = capi.frozen(wrapper)
    assert seen[1] == capi.CRB_ENULL
    assert capi.load() is not None and not isinstance(capi.load(), capi._Recorder)  # the library is back in place
    try:
        call()
    except capi.CrbError as e:
        assert "null operand" in str(e)
    else:
        raise AssertionError("the frozen call did not re-issue crb_sgemm_nn")
    assert len(seen) == 2  # the wrapper itself did not run again
