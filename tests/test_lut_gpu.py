"""Parity of hq_lut_gemv with the CPU oracle (and, where built, the reference's
own kernel), through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, TOL_F16_ACC, rel_err

pytestmark = pytest.mark.gpu


def _run(hq, bW, alpha, qbias, x, group):
    import torch
    dev = torch.device("cuda:0")
    t = lambda a: None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    y = hq.lut_matmul(t(x), t(bW.view(np.int32)), t(alpha), t(qbias), group)
    torch.cuda.synchronize()
    return y.cpu().numpy()


@pytest.mark.parametrize("path", [1, 0])  # 1: matrix-core kernel where the shape allows, 0: table kernel
@pytest.mark.parametrize("K,N,nb,group,zero_bias,seed", [
    (4096, 16384, 3, 128, True, 1), (4096, 16384, 3, 128, False, 2), (1024, 4096, 8, 128, False, 3),
    (1024, 4096, 4, 128, False, 4), (512, 130, 3, 64, False, 5), (96, 64, 1, 32, False, 6),
    (2048, 1001, 2, 2048, False, 7), (1536, 256, 3, 512, False, 8), (640, 192, 5, 128, False, 9),
    (8192, 64, 7, 256, False, 10), (384, 128, 6, 384, False, 11),
    # several rounds per wave (the next round's loads in flight), the last one partly filled
    (12416, 128, 3, 128, False, 28), (16384, 64, 2, 256, True, 29), (5248, 192, 4, 128, False, 30),
    # fewer quads than waves
    (128, 64, 3, 128, False, 31), (256, 64, 1, 256, False, 32), (640, 128, 8, 128, True, 33),
    # group sizes 64 and 32: the grouped matrix-core kernel (N % 64 == 0, K % 128 == 0), every plane count
    (4096, 16384, 3, 64, False, 12), (4096, 4096, 3, 32, False, 13), (1024, 256, 1, 32, False, 14),
    (2048, 128, 2, 64, True, 15), (1152, 192, 4, 32, False, 16), (640, 64, 5, 64, False, 17),
    (896, 128, 6, 32, False, 18), (512, 320, 7, 64, False, 19), (1280, 64, 8, 32, False, 20),
    (128, 64, 3, 32, False, 21), (192, 64, 3, 64, False, 22),
    # N not a multiple of 64 (rows start at any element): the matrix-core kernels with a shifted last tile
    (1024, 1000, 3, 128, False, 23), (512, 72, 4, 64, False, 24), (256, 65, 2, 32, True, 25),
    (4096, 11004, 3, 128, False, 26), (384, 127, 8, 128, False, 27)])
def test_vs_oracle(hq, oracle, tunable, path, K, N, nb, group, zero_bias, seed):
    tunable("HQ_LUT_PATH", path)
    bW, alpha, qbias, x = oa.make_lut_problem(seed, K, N, nb, group, zero_bias)
    y = _run(hq, bW, alpha, qbias, x, group)
    ref = oracle.lut_gemv_f64(bW, alpha, qbias, x, group)
    # fp32 sums rounded once to fp16 (the matrix-core path adds a truncation bias of
    # ~4e-5 of the RMS, a fifth of the fp16 output rounding): far inside the contract
    assert rel_err(y, ref, FLOOR_F16) <= 2e-3
    assert rel_err(y, ref) <= TOL_F16_ACC


@pytest.mark.parametrize("K,N,nb", [(11008, 4096, 3), (8192, 1028, 4), (4224, 448, 8)])
def test_k_split_of_the_plane_kernel(hq, oracle, tunable, K, N, nb):
    """Fewer column tiles than compute units: whole rounds of K go to workgroups of their own, whose partial
    sums the last one to arrive adds in split order.  Same result as the oracle, the same bits on a second
    call and with the formal device-scope fences."""
    bW, alpha, qbias, x = oa.make_lut_problem(50 + nb, K, N, nb, 128, False)
    y = _run(hq, bW, alpha, qbias, x, 128)
    ref = oracle.lut_gemv_f64(bW, alpha, qbias, x, 128)
    assert rel_err(y, ref, FLOOR_F16) <= 2e-3
    assert np.array_equal(y, _run(hq, bW, alpha, qbias, x, 128))
    tunable("HQ_SPLITK_FENCES", 1)
    assert np.array_equal(y, _run(hq, bW, alpha, qbias, x, 128))


def test_plans(hq):
    """Which kernel a shape takes, asked of the library itself: ragged shapes stay on the matrix cores."""
    from hecbench_amd import _lib
    lib = _lib.load()
    TABLE, MFMA, GROUPED, RAGGED = 0, 1, 2, 16
    a16, a4, a2 = 4096, 4100, 4098            # stand-ins for pointers of 16-, 4- and 2-byte alignment
    plan = lambda K, N, nb, G, bw=a16, al=a16, qb=a16: lib.hq_lut_gemv_plan(bw, al, qb, K, N, nb, G)
    assert plan(4096, 16384, 3, 128) == MFMA
    assert plan(4096, 16384, 3, 64) == GROUPED and plan(4096, 4096, 3, 32) == GROUPED
    assert plan(512, 130, 3, 64) == GROUPED | RAGGED
    assert plan(2048, 1001, 2, 2048) == MFMA | RAGGED
    assert plan(4096, 16384, 3, 128, bw=a4) == MFMA | RAGGED       # aligned shape, unaligned operand
    assert plan(4096, 16384, 3, 128, al=a2) == MFMA | RAGGED
    assert plan(4096, 16384, 3, 128, qb=None) == MFMA              # no bias: nothing to align
    assert plan(96, 64, 1, 32) == TABLE                            # K % 128
    assert plan(4096, 48, 3, 128) == TABLE                         # fewer than 64 columns
    assert plan(1536, 256, 3, 96) == TABLE                         # group size 96
    assert plan(4096, 16384, 9, 128) == -2


def test_unaligned_operands(hq, oracle):
    """Operands that start 4 (bit planes) and 2 (alpha, bias) bytes past a 16-byte boundary."""
    import torch
    dev = torch.device("cuda:0")
    K, N, nb, G = 1024, 256, 3, 128
    bW, alpha, qbias, x = oa.make_lut_problem(77, K, N, nb, G, False)
    def shifted(a, dtype, elems):
        buf = torch.zeros(a.size + 16, dtype=dtype, device=dev)
        view = buf[elems:elems + a.size]
        view.copy_(torch.from_numpy(np.ascontiguousarray(a).reshape(-1)).to(dev))
        return view
    dW = shifted(bW.view(np.int32), torch.int32, 1).view(K // 32, nb, N)
    da = shifted(alpha, torch.float16, 1).view(K // G, nb, N)
    dq = shifted(qbias, torch.float16, 3).view(K // G, N)
    assert dW.data_ptr() % 16 == 4 and da.data_ptr() % 16 == 2
    y = hq.lut_matmul(torch.from_numpy(x).to(dev), dW, da, dq, G)
    torch.cuda.synchronize()
    ref = oracle.lut_gemv_f64(bW, alpha, qbias, x, G)
    assert rel_err(y.cpu().numpy(), ref, FLOOR_F16) <= 2e-3


def test_no_bias_pointer(hq, oracle):
    bW, alpha, _, x = oa.make_lut_problem(9, 1024, 512, 3, 128)
    y = _run(hq, bW, alpha, None, x, 128)
    ref = oracle.lut_gemv_f64(bW, alpha, None, x, 128)
    assert rel_err(y, ref, FLOOR_F16) <= 2e-3
    assert rel_err(y, ref) <= TOL_F16_ACC


def test_closed_forms(hq, oracle):
    """alpha = 0 -> y = sum_g bias[g] * sum_{k in g} x;  nb=1, alpha=1, bias=0 -> y = sum +-x."""
    K, N, G = 512, 128, 128
    rng = np.random.default_rng(3)
    x = rng.integers(-4, 5, size=K).astype(np.float16)
    bW = rng.integers(0, 2 ** 32, size=(K // 32, 1, N), dtype=np.uint64).astype(np.uint32)
    qb = rng.integers(-2, 3, size=(K // G, N)).astype(np.float16)
    y = _run(hq, bW, np.zeros((K // G, 1, N), np.float16), qb, x, G)
    want = (qb.astype(np.float64) * x.astype(np.float64).reshape(K // G, G).sum(1)[:, None]).sum(0)
    assert np.array_equal(y.astype(np.float64), want)
    y = _run(hq, bW, np.ones((K // G, 1, N), np.float16), np.zeros((K // G, N), np.float16), x, G)
    bits = ((bW[:, 0, :, None] >> np.arange(32, dtype=np.uint32)) & 1).transpose(0, 2, 1).reshape(K, N)
    want = ((2.0 * bits - 1.0) * x.astype(np.float64)[:, None]).sum(0)
    assert np.array_equal(y.astype(np.float64), want)


def test_vs_reference_kernel(hq, oracle):
    import torch
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built")
    dev = torch.device("cuda:0")
    K, N, nb, G = 4096, 16384, 3, 128
    bW, alpha, qbias, x = oa.make_lut_problem(21, K, N, nb, G, zero_bias=False)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    dW, da, dq, dx = t(bW.view(np.int32)), t(alpha), t(qbias), t(x)
    out = torch.zeros(N, dtype=torch.float16, device=dev)
    vp = lambda a: ctypes.c_void_p(a.data_ptr())
    ref.ref_lut_matmul(vp(out), vp(dx), vp(dW), vp(da), vp(dq), K, N, nb, K // G)
    torch.cuda.synchronize()
    y = hq.lut_matmul(dx, dW, da, dq, G)
    torch.cuda.synchronize()
    r = out.cpu().numpy()
    exact = oracle.lut_gemv_f64(bW, alpha, qbias, x, G)
    # the reference accumulates everything in fp16 (and across 128 K tiles with fp16 atomics)
    assert rel_err(y.cpu().numpy(), r, FLOOR_F16) <= TOL_F16_ACC
    assert rel_err(y.cpu().numpy(), exact) <= rel_err(r, exact)


def test_non_finite_activations_propagate(hq, oracle):
    import torch
    bW, alpha, qb, x = oa.make_lut_problem(55, 1024, 256, 3, 128)
    dev = "cuda:0"
    for bad in (np.nan, np.inf):
        xs = x.copy()
        xs[300] = bad
        y = hq.lut_matmul(torch.from_numpy(xs).to(dev), torch.from_numpy(bW.view(np.int32)).to(dev),
                          torch.from_numpy(alpha).to(dev), torch.from_numpy(qb).to(dev), 128)
        torch.cuda.synchronize()
        assert not np.isfinite(y.cpu().numpy().astype(np.float32)).any(), bad
