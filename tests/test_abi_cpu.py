"""CPU-side checks of the C-ABI library: it is built, loads, and exports every
symbol include/hq.h declares.  No compute call is made (no GPU here)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_bound_and_exported():
    from hecbench_amd import _lib
    declared = _declared_symbols()
    assert declared, "no declarations found in include/hq.h"
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libhq.so not built in this checkout")
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name


def test_strerror_and_version():
    from hecbench_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libhq.so not built in this checkout")
    lib = _lib.load()
    assert lib.hq_abi_version() == 1
    assert b"null pointer" in lib.hq_strerror(-1)
    assert b"shape" in lib.hq_strerror(-2)


def test_argument_validation_needs_no_gpu():
    """Null pointers and bad shapes are rejected before any HIP call."""
    from hecbench_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libhq.so not built in this checkout")
    lib = _lib.load()
    assert lib.hq_q3_matvec(None, 0, None, None, None, None, 4096, 11008, 1, 0, None) == -1
    assert lib.hq_q3_matvec(16, 0, 16, 16, 16, 16, 4095, 11008, 1, 0, None) == -2
    assert lib.hq_q3_matvec(16, 0, 16, 16, 16, 16, 4096, 11006, 1, 0, None) == -2
    assert lib.hq_q3_matvec(16, 7, 16, 16, 16, 16, 4096, 11008, 1, 0, None) == -3
    assert lib.hq_q3_matvec(16, 0, 20, 16, 16, 16, 4096, 11008, 1, 0, None) == -4
    assert lib.hq_q3_matvec(24, 0, 16, 16, 16, 16, 4096, 11008, 1, 0, None) == -4   # x: 128-bit loads
    assert lib.hq_dequant_nf4(None, None, None, 64, 64, 0, None) == -1
    assert lib.hq_dequant_nf4(None, None, None, 0, 64, 0, None) == 0
    assert lib.hq_dequant_nf4(16, 16, 16, 64, 63, 0, None) == -2
    assert lib.hq_dequant_nf4(16, 16, 16, 64, 64, 5, None) == -3
    assert lib.hq_lut_gemv(None, None, None, None, None, 4096, 16384, 3, 128, None) == -1
    assert lib.hq_lut_gemv(16, 16, None, 16, 16, 4096, 16384, 9, 128, None) == -2
    assert lib.hq_lut_gemv(16, 16, None, 16, 16, 4096, 16384, 3, 100, None) == -2
    assert lib.hq_aqlm_matvec(None, None, None, None, None, 4096, 4096, None, 65536, None) == -1
    assert lib.hq_quantize_dynamic8(None, None, None, 5, None) == -1
    assert lib.hq_quantize_dynamic8(None, None, None, 0, None) == 0


def test_tunables_need_no_gpu():
    """Launch-shape knobs are set by name; unknown names and null pointers are rejected."""
    from hecbench_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libhq.so not built in this checkout")
    lib = _lib.load()
    for name in (b"HQ_Q3_WAVES", b"HQ_Q3_STEPS", b"HQ_Q3_KSPLIT", b"HQ_LUT_PATH", b"HQ_NF4_PIPE", b"HQ_AQLM_ROWS",
                 b"HQ_SPLITK_FENCES"):
        assert lib.hq_set_tunable(name, 4, 0) == 0
        assert lib.hq_set_tunable(name, 0, 1) == 0
    assert lib.hq_set_tunable(b"HQ_NO_SUCH_KNOB", 1, 0) == -3
    assert lib.hq_set_tunable(None, 1, 0) == -1
    assert lib.hq_reserve_workspace(None, -1, 0) == -2
