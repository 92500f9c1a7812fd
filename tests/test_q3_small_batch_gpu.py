"""Batches 2 ... 15 of the GPTQ 3-bit product (hq_q3_matvec with batch_M > 1): a batch of 2 runs on the
matvec's digit kernel with the two rows side by side in the matrix-core operand (K split across workgroups
as for batch 1), all others on the batched GEMM.  Every batch size is checked against the CPU oracle through the C ABI,
and the kernel that ran is asserted through hq_q3_matvec_plan.  The reference has no batched kernel:
the oracle is the matvec formula applied row by row (parity unpinned by the reference)."""
import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, rel_err

pytestmark = pytest.mark.gpu

PLAN_MATVEC, PLAN_ROWS, PLAN_GEMM = 0, 1, 2


def _t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def _run(hq, A, mat, scales, zeros):
    import torch
    y = hq.q3_gemm(_t(A), _t(mat), _t(scales), _t(zeros))
    torch.cuda.synchronize()
    return y.cpu().numpy()


def _plan(K, N, M):
    from hecbench_amd import _lib
    return _lib.load().hq_q3_matvec_plan(K, N, M)


def _check(y, exact):
    for m in range(y.shape[0]):
        assert rel_err(y[m], exact[m]) <= 5e-3, m
        assert rel_err(y[m], exact[m], FLOOR_F16) <= 1e-4, m


# wide (N = 257 tiles, the last one 4 columns wide) and narrow (3 tiles, the last one 4 columns wide);
# K = 4128 is not a multiple of a workgroup's round, so the two-row kernel splits it in two;
# the long-K shape is there for the two-row kernel and its neighbours only
_EVERY_BATCH = [(M, K, N) for (K, N) in [(512, 16388), (4128, 8192), (1024, 132)] for M in range(2, 16)
                if K != 4128 or M <= 4]


@pytest.mark.parametrize("M,K,N", _EVERY_BATCH)
def test_every_batch_vs_oracle(hq, oracle, M, K, N):
    codes, scales, zeros, A = oa.make_q3_problem(1000 + 16 * M + (K % 7), K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    want_plan = PLAN_ROWS if M == 2 else PLAN_GEMM
    assert _plan(K, N, M) == want_plan
    y = _run(hq, A, mat, scales, zeros)
    _check(y, oracle.q3_gemm(A, mat, scales, zeros, mode=0))


def test_rows_kernel_against_the_gemm_and_the_matvec(hq, oracle, tunable):
    """The same call with the two-row kernel switched off takes the GEMM; each row also equals the
    batch-1 matvec on that row.  Three kernels, one result (to the accuracy each of them states)."""
    M, K, N = 2, 2048, 16640
    codes, scales, zeros, A = oa.make_q3_problem(500 + M, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, M) == PLAN_ROWS
    y = _run(hq, A, mat, scales, zeros)
    tunable("HQ_Q3_SMALL_BATCH", 0)
    assert _plan(K, N, M) == PLAN_GEMM
    y_gemm = _run(hq, A, mat, scales, zeros)
    for m in range(M):
        assert rel_err(y[m], y_gemm[m]) <= 5e-3
        yv = hq.q3_matvec(_t(A[m]), _t(mat), _t(scales), _t(zeros)).cpu().numpy()
        assert rel_err(y[m], yv) <= 5e-3


@pytest.mark.parametrize("scale_exp", [-16, -8, 0, 4])
def test_rows_kernel_dynamic_range(hq, oracle, scale_exp):
    """Two rows of very different magnitude side by side in one matrix-core operand, an all-zero row, a row
    with one large outlier, magnitudes spread over 2^8 inside a row, fp16 subnormals: every row is held
    to the bound the N(0,1) cases meet, measured against that row's own RMS."""
    K, N = 2048, 8256
    rng = np.random.default_rng(111 + scale_exp)
    codes, scales, zeros, A = oa.make_q3_problem(180 + scale_exp, K, N, x_dtype=np.float16, batch=9)
    mat = oracle.q3_pack(codes)
    A = A.astype(np.float32) * np.float32(2.0 ** scale_exp)
    A[1] *= np.float32(2.0 ** -6)
    A[2] *= np.float32(2.0 ** 5)
    A[4] = 0.0
    A[5, 100] = np.float32(2.0 ** min(15, scale_exp + 12))
    A[6] = rng.standard_normal(K).astype(np.float32) * np.float32(2.0 ** scale_exp) * \
        np.exp2(rng.integers(-8, 1, K)).astype(np.float32)
    A[7, 512:] = 0.0                                       # whole rounds of a wave are zero
    A = A.astype(np.float16)
    for rows in ([0, 1], [2, 4], [3, 5], [6, 7], [4, 8]):
        sub = np.ascontiguousarray(A[rows])
        assert _plan(K, N, len(rows)) == PLAN_ROWS
        y = _run(hq, sub, mat, scales, zeros)
        exact = oracle.q3_gemm(sub, mat, scales, zeros, mode=0)
        for i, m in enumerate(rows):
            if m == 4:
                assert np.all(y[i] == 0.0)
            else:
                assert rel_err(y[i], exact[i]) <= 5e-3, (scale_exp, m)
                assert rel_err(y[i], exact[i], FLOOR_F16) <= 1e-4, (scale_exp, m)


def test_rows_kernel_non_finite_activations(hq, oracle):
    """An infinity or NaN in one row makes that row NaN and leaves the other row alone."""
    K, N = 512, 8192
    codes, scales, zeros, A = oa.make_q3_problem(91, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    A[1, 37] = np.float16(np.inf)
    y = _run(hq, A, mat, scales, zeros)
    exact = oracle.q3_gemm(A[:1], mat, scales, zeros, mode=0)
    assert rel_err(y[0], exact[0]) <= 5e-3
    assert np.all(np.isnan(y[1]))


def test_config4_shape_batches_2_and_3(hq, oracle):
    """K=8192, N=28672 (the GEMM configuration's weights) at batch 2 (two-row kernel) and 3 (GEMM): sampled
    columns against the oracle, all columns against the batch-1 matvec."""
    import torch
    K, N = 8192, 28672
    rng = np.random.default_rng(45)
    mat = rng.integers(-2 ** 31, 2 ** 31, size=(3 * K // 32, N), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, size=N).astype(np.float32)
    zeros = (scales * rng.integers(3, 5, size=N)).astype(np.float32)
    dm, ds, dz = _t(mat), _t(scales), _t(zeros)
    cols = np.unique(np.concatenate([np.arange(0, 132), np.arange(N - 132, N), rng.integers(0, N, 120)]))
    sub = np.ascontiguousarray(mat[:, cols])
    for M in (2, 3):
        A = rng.standard_normal((M, K)).astype(np.float16)
        assert _plan(K, N, M) == (PLAN_ROWS if M == 2 else PLAN_GEMM)
        y = hq.q3_gemm(_t(A), dm, ds, dz)
        torch.cuda.synchronize()
        y = y.cpu().numpy()
        _check(y[:, cols], oracle.q3_gemm(A, sub, scales[cols], zeros[cols], mode=0))
        for m in range(M):
            yv = hq.q3_matvec(_t(A[m]), dm, ds, dz).cpu().numpy()
            assert rel_err(y[m], yv) <= 5e-3


def test_rows_kernel_accumulates(hq, oracle):
    """HQ_FLAG_ACCUMULATE adds to what y holds, as for batch 1."""
    import torch
    from hecbench_amd import _lib
    M, K, N = 2, 256, 8196
    codes, scales, zeros, A = oa.make_q3_problem(300 + M, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    rng = np.random.default_rng(5)
    y0 = rng.standard_normal((M, N)).astype(np.float32)
    dA, dm, ds, dz, dy = _t(A), _t(mat), _t(scales), _t(zeros), _t(y0)
    assert _plan(K, N, M) == PLAN_ROWS
    rc = _lib.load().hq_q3_matvec(dA.data_ptr(), 1, dm.data_ptr(), ds.data_ptr(), dz.data_ptr(), dy.data_ptr(),
                                  K, N, M, 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    got = dy.cpu().numpy() - y0
    for m in range(M):
        assert rel_err(got[m], exact[m], FLOOR_F16) <= 1e-3   # y0 ~ 1 costs a few fp32 ulps of it


@pytest.mark.parametrize("K", [32, 96, 160])
def test_rows_kernel_short_k(hq, oracle, K):
    """Fewer k-groups than a workgroup's waves cover: idle waves, partly filled steps."""
    N = 8200
    codes, scales, zeros, A = oa.make_q3_problem(700 + K, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, 2) == PLAN_ROWS
    _check(_run(hq, A, mat, scales, zeros), oracle.q3_gemm(A, mat, scales, zeros, mode=0))


# (K, N, forced split or 0): K rounds of 4096 -> one workgroup per round up to eight (three for K = 11008,
# the last one partly filled), beyond that as many workgroups per tile as the compute units allow, each
# walking several rounds (K = 36864, 64 tiles); a forced single workgroup walks all of K in rounds
_SPLIT_SHAPES = [(11008, 4096, 0), (36864, 4096, 0), (40960, 1028, 0), (11008, 4096, 1), (8192, 260, 2)]


@pytest.mark.parametrize("K,N,force", _SPLIT_SHAPES)
def test_rows_kernel_splits_k(hq, oracle, tunable, K, N, force):
    """Partial sums of both rows per workgroup, added by the last one to arrive: same result as the
    oracle, the same bits on a second call (the counters reset themselves), and as the batch-1 matvec."""
    codes, scales, zeros, A = oa.make_q3_problem(900 + K % 97 + N % 13, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    if force:
        tunable("HQ_Q3_KSPLIT", force)
    assert _plan(K, N, 2) == PLAN_ROWS
    y = _run(hq, A, mat, scales, zeros)
    _check(y, oracle.q3_gemm(A, mat, scales, zeros, mode=0))
    assert np.array_equal(_run(hq, A, mat, scales, zeros), y)
    for m in range(2):
        yv = hq.q3_matvec(_t(A[m]), _t(mat), _t(scales), _t(zeros)).cpu().numpy()
        assert rel_err(y[m], yv) <= 5e-3


def test_rows_kernel_split_k_accumulates_and_strict_fences(hq, oracle, tunable):
    import torch
    from hecbench_amd import _lib
    M, K, N = 2, 12288, 2052
    codes, scales, zeros, A = oa.make_q3_problem(333, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    y0 = np.random.default_rng(6).standard_normal((M, N)).astype(np.float32)
    dA, dm, ds, dz = _t(A), _t(mat), _t(scales), _t(zeros)
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    plain = _run(hq, A, mat, scales, zeros)
    for strict in (0, 1):
        tunable("HQ_SPLITK_FENCES", strict)
        dy = _t(y0)
        rc = _lib.load().hq_q3_matvec(dA.data_ptr(), 1, dm.data_ptr(), ds.data_ptr(), dz.data_ptr(), dy.data_ptr(),
                                      K, N, M, 1, None)
        assert rc == 0
        torch.cuda.synchronize()
        got = dy.cpu().numpy()
        assert np.array_equal(got, y0 + plain)   # one fp32 addition to the finished sum
        for m in range(M):
            assert rel_err(got[m] - y0[m], exact[m], FLOOR_F16) <= 1e-3
