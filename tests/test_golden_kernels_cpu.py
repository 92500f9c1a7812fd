"""The oracle against golden outputs of the reference's own DEVICE kernels (tests/golden/*.npz,
written on an MI355X by tests/golden/make_golden_gpu.py from the reference compiled out of its own
sources).  Runs without a GPU and without the reference tree."""
import os

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, TOL_F16_ACC, TOL_F32_ACC, rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def o():
    return oa.load_oracle()


def _load(name):
    path = os.path.join(GOLDEN, name)
    if not os.path.exists(path):
        pytest.skip(f"{name} not present")
    return np.load(path)


def test_mxfp4_matches_reference_kernel_bit_for_bit(o):
    g = _load("mxfp4_reference_kernel.npz")
    for name, bf16 in (("f16", False), ("bf16", True)):
        got = o.mxfp4_qdq(g[f"in_{name}"], bf16)
        want = g[f"out_{name}"]
        # groups whose maximum rounds to zero are where the reference divides by a zero scale
        live = np.repeat((g[f"in_{name}"].reshape(-1, 32) & 0x7fff).max(axis=1) >= (0x0080 if bf16 else 0x0400), 32)
        assert live.mean() > 0.99
        assert np.array_equal(got[live], want[live]), name


def test_gemv_within_fp16_rounding_of_reference_kernels(o):
    g = _load("gemv_reference_kernels.npz")
    for mode, name in ((0, "fp16"), (1, "int8"), (2, "int4")):
        r16, r64 = o.gemv(g[f"mat_{name}"], mode, g[f"vec_{name}"], 0.0625, 0.01)
        theirs = g[f"res_{name}"].astype(np.float64)
        # the reference kernels sum in fp32 in a thread-dependent order and round once to fp16
        rms = np.sqrt(np.mean(r64 ** 2))
        assert np.all(np.abs(theirs - r64) <= np.abs(r64) * 2.0 ** -10 + 1e-4 * rms), name


def test_q3_matvec_vs_reference_kernels(o):
    g = _load("q3_reference_kernels.npz")
    mat, s, z, x = g["mat"], g["scales"], g["zeros"], g["x"]
    ref64 = o.q3_matvec_f64(x, mat, s, z)
    assert rel_err(g["y_f32_kernel"], ref64) <= TOL_F32_ACC
    assert rel_err(o.q3_matvec_f32(x, mat, s, z), g["y_f32_kernel"]) <= 1e-4     # same arithmetic, other block order
    y16 = o.q3_matvec_f16(x.astype(np.float16), mat, s, z)
    assert rel_err(y16, g["y_faster_kernel"], FLOOR_F16) <= 2e-3                 # fp16 restatement vs the real kernel
    assert rel_err(g["y_faster_kernel"], ref64, FLOOR_F16) <= TOL_F16_ACC


def test_aqlm_restatement_is_bit_identical_to_reference_kernel(o):
    g = _load("aqlm_reference_kernel.npz")
    cb = np.zeros((2, 65536, 8), np.float16)
    cb[:, g["used_entries"], :] = g["used_values"]
    y16, _ = o.aqlm_matvec(g["codes"], cb, None, g["x"], tuple(int(v) for v in g["sizes"]), 65536, mode=1)
    assert np.array_equal(y16.view(np.uint16), g["y"].view(np.uint16))
    y_exact, y64 = o.aqlm_matvec(g["codes"], cb, None, g["x"], tuple(int(v) for v in g["sizes"]), 65536, mode=0)
    assert rel_err(g["y"], y64, FLOOR_F16) <= TOL_F16_ACC


def test_int8_quantisers_equal_reference_kernels(o):
    import torch
    g = _load("quantvllm_reference_kernels.npz")
    for name in ("f32", "f16", "bf16"):
        x = g[f"x_{name}"]
        if name == "bf16":
            x = torch.from_numpy(x.view(np.int16).copy()).view(torch.bfloat16)
        for azp in (0, 54):
            assert np.array_equal(o.int8_quant_static(x, 0.1, azp if azp else None), g[f"static_{name}_azp{azp}"])
        for with_azp in (0, 1):
            q, sc, zp = o.int8_quant_dynamic(x, bool(with_azp))
            assert np.array_equal(q, g[f"dynamic_{name}_azp{with_azp}"])
            assert np.array_equal(sc, g[f"dynamic_{name}_azp{with_azp}_scales"])
            if with_azp:
                assert np.array_equal(zp, g[f"dynamic_{name}_azp1_zero_points"])


def test_quantize_dynamic8_equals_reference_kernel(o):
    g = _load("kquantize_reference_kernel.npz")
    assert np.array_equal(o.quantize_dynamic8(g["code"], g["A"]), g["out"])
