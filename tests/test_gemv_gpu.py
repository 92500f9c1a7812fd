"""Parity of the dense / int8 / int4 matrix-vector products with the CPU oracle and, where it was
built, with the reference kernels themselves (same device buffers), through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.test_gemv_mxfp4_cpu import gemv_problem

pytestmark = pytest.mark.gpu

SCALE, ZP = 0.0625, 0.01     # the reference's default -u / -v (src/gemv-hip/main.cu:35-36)


def _run(hq, mat, vec, mode):
    import torch
    dm = torch.from_numpy(mat).to("cuda:0")
    dv = torch.from_numpy(vec).to("cuda:0")
    if mode == 0:
        out = hq.gemv_fp16(dm, dv)
    elif mode == 1:
        out = hq.gemv_int8(dm, dv, SCALE, ZP)
    else:
        out = hq.gemv_int4(dm, dv, SCALE, ZP)
    torch.cuda.synchronize()
    return out.cpu().numpy(), dm, dv


def _check(got16, ref64):
    # one rounding to fp16 (half an ulp, 2^-11 relative) on top of fp32 sums whose error is a few
    # 1e-6 of the typical output size
    got = got16.astype(np.float64)
    rms = float(np.sqrt(np.mean(ref64 ** 2)))
    bound = np.abs(ref64) * 2.0 ** -10 + 1e-5 * rms + 2.0 ** -24
    assert np.all(np.abs(got - ref64) <= bound), float(np.max(np.abs(got - ref64) / bound))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("rows,n", [(512, 512), (37, 1024), (1, 32), (9000, 2048), (3, 16384), (130, 96), (16390, 64)])
def test_vs_oracle(hq, oracle, rows, n, mode):
    mat, vec = gemv_problem(rows + n + mode, rows, n, mode)
    got, _, _ = _run(hq, mat, vec, mode)
    _, r64 = oracle.gemv(mat, mode, vec, SCALE, ZP)
    _check(got, r64)


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("rows,n", [(512, 512), (37, 1024), (1, 32), (9000, 2048), (16390, 64), (4099, 4096),
                                    (16385, 1056), (40, 65536)])
def test_vector_in_lds_kernel(hq, oracle, tunable, rows, n, mode):
    """The persistent kernel that keeps the vector in LDS (by default only int4 with many rows), forced on
    shapes with one, two and four rows per wave, ragged row counts, rows shorter than one step of a wave
    and the longest vector it takes; and the ordinary kernel forced where the rule would pick the other:
    both must give the same bits, and the oracle's result."""
    import torch
    mat, vec = gemv_problem(rows * 3 + n + mode, rows, n, mode)
    _, r64 = oracle.gemv(mat, mode, vec, SCALE, ZP)
    tunable("HQ_GEMV_LDS", 1)
    lds, _, _ = _run(hq, mat, vec, mode)
    _check(lds, r64)
    tunable("HQ_GEMV_LDS", 0)
    plain, _, _ = _run(hq, mat, vec, mode)
    assert np.array_equal(lds.view(np.uint16), plain.view(np.uint16))


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("split", [4, 8, 16])
@pytest.mark.parametrize("rows,n", [(37, 1024), (1, 32), (513, 8192), (16, 16384), (131, 11008), (7, 65536 + 64)])
def test_rows_cut_across_waves(hq, oracle, tunable, rows, n, mode, split):
    """The kernel whose workgroups share a pair of rows, every wave a piece of the columns: forced with 4, 8
    and 16 waves on odd row counts, rows shorter than one step per wave (idle waves) and rows that do not
    divide into whole steps."""
    mat, vec = gemv_problem(rows * 7 + n + mode + split, rows, n, mode)
    _, r64 = oracle.gemv(mat, mode, vec, SCALE, ZP)
    tunable("HQ_GEMV_SPLIT", split)
    got, _, _ = _run(hq, mat, vec, mode)
    _check(got, r64)


@pytest.mark.parametrize("rows,n", [(130, 8192), (33, 16384), (66, 28672), (5, 32768)])
def test_long_fp16_rows_default_rule(hq, oracle, rows, n):
    """fp16 rows of 8192 elements or more take the split kernel by default."""
    mat, vec = gemv_problem(rows + n, rows, n, 0)
    _, r64 = oracle.gemv(mat, 0, vec, SCALE, ZP)
    got, _, _ = _run(hq, mat, vec, 0)
    _check(got, r64)


def test_vector_too_long_for_lds(hq, oracle, tunable):
    """Beyond 65536 elements the vector does not fit: the ordinary kernel runs even when the other is asked for."""
    mat, vec = gemv_problem(5, 24, 65536 + 32, 2)
    tunable("HQ_GEMV_LDS", 1)
    got, _, _ = _run(hq, mat, vec, 2)
    _, r64 = oracle.gemv(mat, 2, vec, SCALE, ZP)
    _check(got, r64)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_signed_data_and_extremes(hq, oracle, mode):
    """Signed vector entries (cancellation) and the extreme codes -128 / 127 / 0 / 15."""
    rng = np.random.default_rng(3)
    rows, n = 64, 4096
    vec = rng.standard_normal(n).astype(np.float16)
    if mode == 0:
        mat = rng.standard_normal((rows, n)).astype(np.float16)
    elif mode == 1:
        mat = rng.choice(np.array([-128, 127, 0, 1], np.int8), (rows, n))
    else:
        mat = rng.choice(np.array([0x00, 0xFF, 0xF0, 0x0F], np.uint8), (rows, n // 2))
    got, _, _ = _run(hq, mat, vec, mode)
    _, r64 = oracle.gemv(mat, mode, vec, SCALE, ZP)
    # zero-mean sums: error relative to the size of the terms, not of the (cancelled) result
    dense = np.abs(mat.astype(np.float64)).max() if mode != 2 else 15.0
    scale = np.sqrt(n) * dense * (SCALE if mode else 1.0)
    assert np.max(np.abs(got.astype(np.float64) - r64)) <= 2e-3 * scale


def test_rejects_bad_arguments(hq):
    import torch
    from hecbench_amd import HqError
    v = torch.zeros(40, dtype=torch.float16, device="cuda:0")
    with pytest.raises(HqError):
        hq.gemv_fp16(torch.zeros(4, 36, dtype=torch.float16, device="cuda:0"), v[:36])     # n % 8
    with pytest.raises(HqError):
        hq.gemv_int8(torch.zeros(4, 40, dtype=torch.int8, device="cuda:0"), v, 1.0, 0.0)   # n % 16
    with pytest.raises(HqError):
        hq.gemv_int4(torch.zeros(4, 20, dtype=torch.uint8, device="cuda:0"), v, 1.0, 0.0)  # n % 32


@pytest.mark.parametrize("n,bx,by", [(512, 32, 4), (2048, 128, 8)])
def test_vs_reference_kernels(hq, oracle, n, bx, by):
    """The reference's three kernels on the same device buffers, with the launch shapes of its run
    lines (src/gemv-hip/Makefile:55-57): both sides within the reference's own acceptance band
    (0.125 * n / 512, gemv.cu:143) of each other and of the exact result."""
    import torch
    ref = oa.load_ref_hip()
    if ref is None or not hasattr(ref, "ref_gemv_fp16"):
        pytest.skip("oracle/_ref was not built with the gemv kernels")
    vp = ctypes.c_void_p
    for mode in (0, 1, 2):
        mat, vec = gemv_problem(11 * mode + n, n, n, mode)
        got, dm, dv = _run(hq, mat, vec, mode)
        res = torch.zeros(n, dtype=torch.float16, device="cuda:0")
        args = [vp(dm.data_ptr()), vp(dv.data_ptr()), vp(res.data_ptr()), ctypes.c_uint(n)]
        if mode == 0:
            ref.ref_gemv_fp16(*args, ctypes.c_uint(bx), ctypes.c_uint(by), None)
        else:
            fn = ref.ref_gemv_int8 if mode == 1 else ref.ref_gemv_int4
            fn(*args, ctypes.c_float(SCALE), ctypes.c_float(ZP), ctypes.c_uint(bx), ctypes.c_uint(by), None)
        torch.cuda.synchronize()
        theirs = res.cpu().numpy().astype(np.float64)
        _, r64 = oracle.gemv(mat, mode, vec, SCALE, ZP)
        band = 0.125 * n / 512
        assert np.max(np.abs(theirs - r64)) <= band
        assert np.max(np.abs(got.astype(np.float64) - theirs)) <= band
        # and this library is at least as close to the exact result as the reference kernel
        assert np.max(np.abs(got.astype(np.float64) - r64)) <= np.max(np.abs(theirs - r64)) + 1e-6
