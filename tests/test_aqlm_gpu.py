"""Parity of hq_aqlm_matvec with the CPU oracle (and, where built, the
reference's own kernel), through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, TOL_F16_ACC, rel_err

pytestmark = pytest.mark.gpu


def _run(hq, codes, codebooks, scales, x, sizes, stride=65536):
    import torch
    dev = torch.device("cuda:0")
    t = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    y = hq.code1x16_matvec(t(codes), t(x), t(codebooks), sizes, stride, scales=t(scales))
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("M,K,seed", [(4096, 4096, 1), (64, 256, 2), (1000, 1024, 3), (7, 8192, 4), (3, 64, 5)])
def test_vs_oracle(hq, oracle, M, K, seed):
    codes, cb, scales, x = oa.make_aqlm_problem(seed, M, K)
    y = _run(hq, codes, cb, scales, x, (M, 0, 0, 0))
    _, ref64 = oracle.aqlm_matvec(codes, cb, scales, x, (M, 0, 0, 0), 65536, mode=0)
    assert rel_err(y, ref64) <= 2e-3
    ref16, _ = oracle.aqlm_matvec(codes, cb, scales, x, (M, 0, 0, 0), 65536, mode=1)
    assert rel_err(y, ref16.astype(np.float64), FLOOR_F16) <= TOL_F16_ACC


def test_three_codebooks_and_no_scale(hq, oracle):
    """Reference default geometry: 3 code books of 4096 rows each, no scale."""
    M, K = 12288, 1024
    codes, cb, _, x = oa.make_aqlm_problem(11, M, K, ncb=3)
    sizes = (4096, 8192, 12288, 122880)
    y = _run(hq, codes, cb, None, x, sizes)
    _, ref64 = oracle.aqlm_matvec(codes, cb, None, x, sizes, 65536, mode=0)
    assert rel_err(y, ref64) <= 2e-3
    # partition boundaries: constant code books make the row's code book visible
    cbc = np.zeros((3, 65536, 8), np.float16)
    cbc[0], cbc[1], cbc[2] = 1.0, 2.0, 3.0
    xs = np.ones(K, np.float16) / 8
    y = _run(hq, codes, cbc, None, xs, sizes)
    assert (y[:4096] == K / 8).all() and (y[4096:8192] == 2 * K / 8).all() and (y[8192:] == 3 * K / 8).all()


def test_signed_codes_and_gather(hq, oracle):
    """-1 -> entry 65535, -32768 -> entry 32768; one-hot entries gather x."""
    M, K = 4, 64
    cb = np.zeros((1, 65536, 8), np.float16)
    cb[0, 65535, 0] = 1.0
    cb[0, 32768, 7] = 1.0
    cb[0, 5, 3] = 1.0
    codes = np.zeros((M, K // 8), np.int16)
    codes[0, :] = -1
    codes[1, :] = -32768
    codes[2, :] = 5
    x = (np.arange(K) + 1).astype(np.float16)
    y = _run(hq, codes, cb, None, x, (M, 0, 0, 0))
    assert y[0] == x[0::8].astype(np.float64).sum()
    assert y[1] == x[7::8].astype(np.float64).sum()
    assert y[2] == x[3::8].astype(np.float64).sum()
    assert y[3] == 0


def test_vs_reference_kernel(hq, oracle):
    import torch
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built")
    dev = torch.device("cuda:0")
    M, K = 12288, 4096
    codes, cb, _, x = oa.make_aqlm_problem(31, M, K, ncb=3)
    sizes = (4096, 8192, 12288, 122880)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    dc, dcb, dx = t(codes), t(cb), t(x)
    out = torch.zeros(M, dtype=torch.float16, device=dev)
    vp = lambda a: ctypes.c_void_p(a.data_ptr())
    ref.ref_code1x16_launch(vp(dc), vp(dx), vp(out), vp(dcb), M, K, (ctypes.c_int * 4)(*sizes), 65536, None)
    torch.cuda.synchronize()
    y = hq.code1x16_matvec(dc, dx, dcb, sizes, 65536)
    torch.cuda.synchronize()
    r = out.cpu().numpy()
    assert rel_err(y.cpu().numpy(), r, FLOOR_F16) <= TOL_F16_ACC
    # the oracle's restatement of the reference arithmetic matches the real kernel bit for bit
    ref16, _ = oracle.aqlm_matvec(codes[:256], cb, None, x, sizes, 65536, mode=1)
    assert np.array_equal(ref16.view(np.uint16), r[:256].view(np.uint16))
