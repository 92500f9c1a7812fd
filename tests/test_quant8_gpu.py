"""Bit-exact parity of hq_quantize_dynamic8 with the CPU oracle, through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def _run(hq, code, A):
    import torch
    dev = torch.device("cuda:0")
    out = hq.quantize_dynamic8(torch.from_numpy(code).to(dev), torch.from_numpy(A).to(dev))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("n", [1 << 20, 1000003, 5, 256])
def test_bit_exact_normal_inputs(hq, oracle, n):
    code = oracle.dynamic_map()
    A = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    assert np.array_equal(_run(hq, code, A), oracle.quantize_dynamic8(code, A))


def test_table_values_midpoints_and_extremes(hq, oracle):
    code = oracle.dynamic_map()
    mids = ((code[:-1].astype(np.float64) + code[1:]) / 2).astype(np.float32)
    A = np.concatenate([code, mids, np.nextafter(mids, np.float32(2)), np.nextafter(mids, np.float32(-2)),
                        np.array([-5, 5, -1, 1, 0, -0.0, 1e-30, -1e-30, np.inf, -np.inf], np.float32)])
    assert np.array_equal(_run(hq, code, A), oracle.quantize_dynamic8(code, A))


def test_vs_reference_kernel(hq, oracle):
    import torch
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built")
    dev = torch.device("cuda:0")
    ref.ref_hip_code_table.restype = ctypes.POINTER(ctypes.c_float)
    code = np.ctypeslib.as_array(ref.ref_hip_code_table(), shape=(256,)).copy()
    n = 1 << 20
    A = np.random.default_rng(77).standard_normal(n).astype(np.float32)
    dA, dcode = torch.from_numpy(A).to(dev), torch.from_numpy(code).to(dev)
    out = torch.zeros(n, dtype=torch.uint8, device=dev)
    ref.ref_kquantize(ctypes.c_void_p(dcode.data_ptr()), ctypes.c_void_p(dA.data_ptr()),
                      ctypes.c_void_p(out.data_ptr()), ctypes.c_long(n), None)
    torch.cuda.synchronize()
    y = hq.quantize_dynamic8(dcode, dA)
    torch.cuda.synchronize()
    assert torch.equal(y, out)
