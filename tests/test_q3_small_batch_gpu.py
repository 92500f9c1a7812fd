"""Batches 2 ... 16 of the GPTQ 3-bit product (hq_q3_matvec with batch_M > 1): batches 2 ... 8 (up to 12 on
small launches) run on the matvec's matrix-core kernel with every activation as four small fp8 terms under
one scale per 32 activations (four rows side by side in the operand per pass over the weights, K split across
workgroups as for batch 1), all others on the batched GEMM.  Every batch size is checked against the CPU oracle through the C ABI,
and the kernel that ran is asserted through hq_q3_matvec_plan.  The reference has no batched kernel:
the oracle is the matvec formula applied row by row (parity unpinned by the reference)."""
import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, rel_err

pytestmark = pytest.mark.gpu

PLAN_MATVEC, PLAN_GEMM, PLAN_BLOCK = 0, 2, 3


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
# K = 4128 is not a multiple of a workgroup's round, so the kernel splits it in two;
# the long-K shape is there for the smallest batches only
_EVERY_BATCH = [(M, K, N) for (K, N) in [(512, 16388), (4128, 8192), (1024, 132)] for M in list(range(2, 35)) + [47, 48, 61, 64, 65, 66]
                if (K == 512 and M <= 15) or (K == 4128 and M <= 4) or K == 1024]


@pytest.mark.parametrize("M,K,N", _EVERY_BATCH)
def test_every_batch_vs_oracle(hq, oracle, M, K, N):
    codes, scales, zeros, A = oa.make_q3_problem(1000 + 16 * M + (K % 7), K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    # more than four rows: row blocks of four where that makes at most four workgroups per compute unit (the
    # wide shape: up to three blocks of its 257 tiles), up to 64 rows
    want_plan = PLAN_BLOCK if M <= (12 if N > 1000 else 64) else PLAN_GEMM
    assert _plan(K, N, M) == want_plan
    y = _run(hq, A, mat, scales, zeros)
    _check(y, oracle.q3_gemm(A, mat, scales, zeros, mode=0))


def test_batch2_against_the_gemm_and_the_matvec(hq, oracle, tunable):
    """The same call with the small-batch kernel switched off takes the GEMM; each row also equals the
    batch-1 matvec on that row.  Three kernels, one result (to the accuracy each of them states)."""
    M, K, N = 2, 2048, 16640
    codes, scales, zeros, A = oa.make_q3_problem(500 + M, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, M) == PLAN_BLOCK
    y = _run(hq, A, mat, scales, zeros)
    tunable("HQ_Q3_SMALL_BATCH", 0)
    assert _plan(K, N, M) == PLAN_GEMM
    y_gemm = _run(hq, A, mat, scales, zeros)
    for m in range(M):
        assert rel_err(y[m], y_gemm[m]) <= 5e-3
        yv = hq.q3_matvec(_t(A[m]), _t(mat), _t(scales), _t(zeros)).cpu().numpy()
        assert rel_err(y[m], yv) <= 5e-3


@pytest.mark.parametrize("scale_exp", [-16, -8, 0, 4])
def test_batch2_dynamic_range(hq, oracle, scale_exp):
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
        assert _plan(K, N, len(rows)) == PLAN_BLOCK
        y = _run(hq, sub, mat, scales, zeros)
        exact = oracle.q3_gemm(sub, mat, scales, zeros, mode=0)
        for i, m in enumerate(rows):
            if m == 4:
                assert np.all(y[i] == 0.0)
            else:
                assert rel_err(y[i], exact[i]) <= 5e-3, (scale_exp, m)
                assert rel_err(y[i], exact[i], FLOOR_F16) <= 1e-4, (scale_exp, m)


def test_batch2_non_finite_activations(hq, oracle):
    """An infinity or NaN in one row makes that row NaN and leaves the other row alone."""
    K, N = 512, 8192
    codes, scales, zeros, A = oa.make_q3_problem(91, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    A[1, 37] = np.float16(np.inf)
    y = _run(hq, A, mat, scales, zeros)
    exact = oracle.q3_gemm(A[:1], mat, scales, zeros, mode=0)
    assert rel_err(y[0], exact[0]) <= 5e-3
    assert np.all(np.isnan(y[1]))


def test_config4_shape_batches_2_3_and_11(hq, oracle):
    """K=8192, N=28672 (the GEMM configuration's weights) at batches 2 and 3 (four rows per pass)
    and 11 (GEMM): sampled columns against the oracle, all columns against the batch-1 matvec."""
    import torch
    K, N = 8192, 28672
    rng = np.random.default_rng(45)
    mat = rng.integers(-2 ** 31, 2 ** 31, size=(3 * K // 32, N), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, size=N).astype(np.float32)
    zeros = (scales * rng.integers(3, 5, size=N)).astype(np.float32)
    dm, ds, dz = _t(mat), _t(scales), _t(zeros)
    cols = np.unique(np.concatenate([np.arange(0, 132), np.arange(N - 132, N), rng.integers(0, N, 120)]))
    sub = np.ascontiguousarray(mat[:, cols])
    for M in (2, 3, 11):
        A = rng.standard_normal((M, K)).astype(np.float16)
        assert _plan(K, N, M) == {2: PLAN_BLOCK, 3: PLAN_BLOCK, 11: PLAN_GEMM}[M]
        y = hq.q3_gemm(_t(A), dm, ds, dz)
        torch.cuda.synchronize()
        y = y.cpu().numpy()
        _check(y[:, cols], oracle.q3_gemm(A, sub, scales[cols], zeros[cols], mode=0))
        for m in range(M):
            yv = hq.q3_matvec(_t(A[m]), dm, ds, dz).cpu().numpy()
            assert rel_err(y[m], yv) <= 5e-3


def test_batch2_accumulates(hq, oracle):
    """HQ_FLAG_ACCUMULATE adds to what y holds, as for batch 1."""
    import torch
    from hecbench_amd import _lib
    M, K, N = 2, 256, 8196
    codes, scales, zeros, A = oa.make_q3_problem(300 + M, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    rng = np.random.default_rng(5)
    y0 = rng.standard_normal((M, N)).astype(np.float32)
    dA, dm, ds, dz, dy = _t(A), _t(mat), _t(scales), _t(zeros), _t(y0)
    assert _plan(K, N, M) == PLAN_BLOCK
    rc = _lib.load().hq_q3_matvec(dA.data_ptr(), 1, dm.data_ptr(), ds.data_ptr(), dz.data_ptr(), dy.data_ptr(),
                                  K, N, M, 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    got = dy.cpu().numpy() - y0
    for m in range(M):
        assert rel_err(got[m], exact[m], FLOOR_F16) <= 1e-3   # y0 ~ 1 costs a few fp32 ulps of it


@pytest.mark.parametrize("K", [32, 96, 160])
def test_batch2_short_k(hq, oracle, K):
    """Fewer k-groups than a workgroup's waves cover: idle waves, partly filled steps."""
    N = 8200
    codes, scales, zeros, A = oa.make_q3_problem(700 + K, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, 2) == PLAN_BLOCK
    _check(_run(hq, A, mat, scales, zeros), oracle.q3_gemm(A, mat, scales, zeros, mode=0))


# K rounds of 4096 -> one workgroup per round up to eight (three for K = 11008, the last one partly filled),
# beyond that as many workgroups per tile as give every compute unit two, each walking several rounds
_SPLIT_SHAPES = [(11008, 4096), (36864, 4096), (40960, 1028), (8192, 260)]


@pytest.mark.parametrize("K,N", _SPLIT_SHAPES)
def test_batch2_splits_k(hq, oracle, K, N):
    """Partial sums of both rows per workgroup, added by the last one to arrive: same result as the
    oracle, the same bits on a second call (the counters reset themselves), and as the batch-1 matvec."""
    codes, scales, zeros, A = oa.make_q3_problem(900 + K % 97 + N % 13, K, N, x_dtype=np.float16, batch=2)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, 2) == PLAN_BLOCK
    y = _run(hq, A, mat, scales, zeros)
    _check(y, oracle.q3_gemm(A, mat, scales, zeros, mode=0))
    assert np.array_equal(_run(hq, A, mat, scales, zeros), y)
    for m in range(2):
        yv = hq.q3_matvec(_t(A[m]), _t(mat), _t(scales), _t(zeros)).cpu().numpy()
        assert rel_err(y[m], yv) <= 5e-3


def test_batch2_split_k_accumulates_and_strict_fences(hq, oracle, tunable):
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


@pytest.mark.parametrize("M,K,N", [(M, K, N) for (K, N) in [(1024, 196), (4128, 8192)] for M in (2, 3, 4, 5, 8, 11)])
def test_small_batches_on_the_gemm(hq, oracle, tunable, M, K, N):
    """HQ_Q3_SMALL_BATCH=0 keeps the digit kernels out: the GEMM serves the small batches as well."""
    tunable("HQ_Q3_SMALL_BATCH", 0)
    assert _plan(K, N, M) == PLAN_GEMM
    codes, scales, zeros, A = oa.make_q3_problem(1300 + M, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    _check(_run(hq, A, mat, scales, zeros), oracle.q3_gemm(A, mat, scales, zeros, mode=0))


# one and two passes of four rows, full and partly filled; K of one round, a K the rounds do not divide
# (two workgroups per tile), eight rounds, and more (workgroups that take several rounds, the last one partly
# filled); N with a 4-column last tile
_BLOCK_CASES = [(M, K, N) for (K, N) in [(4128, 1028), (160, 16388)] for M in (3, 4, 5, 6, 7, 8)] + \
               [(6, 32768, 260), (8, 16384, 196), (4, 8192, 4096), (4, 36864, 1028), (3, 49184, 260)] + \
               [(M, K, N) for (K, N) in [(4128, 1028), (512, 4100)] for M in (9, 10, 11, 12)]


@pytest.mark.parametrize("M,K,N", _BLOCK_CASES)
def test_block_kernel_vs_oracle(hq, oracle, M, K, N):
    """Four rows per pass, four fp8 terms per activation: against the oracle at the batch-1 kernel's bound
    (N(0,1) activations enter exactly) and, row by row, the batch-1 matvec; a second call gives the same bits
    (partial sums and counters are left ready)."""
    assert _plan(K, N, M) == PLAN_BLOCK
    codes, scales, zeros, A = oa.make_q3_problem(1500 + 16 * M + K % 11, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    y = _run(hq, A, mat, scales, zeros)
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    for m in range(M):
        assert rel_err(y[m], exact[m]) <= 1e-3, m
    assert np.array_equal(_run(hq, A, mat, scales, zeros), y)
    dm, ds, dz = _t(mat), _t(scales), _t(zeros)
    for m in (0, M - 1):
        yv = hq.q3_matvec(_t(A[m]), dm, ds, dz).cpu().numpy()
        assert rel_err(y[m], yv) <= 1e-3


@pytest.mark.parametrize("M,K,N", [(5, 4128, 1028), (8, 512, 4100), (11, 4128, 1028), (12, 160, 16388), (13, 1024, 132),
                                   (16, 8192, 260), (23, 4096, 516), (32, 32768, 68), (32, 160, 4100), (61, 4128, 260), (64, 512, 132)])
def test_row_blocks_and_passes_agree(hq, oracle, tunable, M, K, N):
    """More than four rows as row blocks of four (one workgroup each; forced here whatever the launch size, with
    and without a K split, with a last block of one to four rows) against the oracle, against the same batch
    as passes of one workgroup (up to twelve rows) and, row by row, against the batch-1 matvec."""
    codes, scales, zeros, A = oa.make_q3_problem(1700 + 16 * M + K % 13, K, N, x_dtype=np.float16, batch=M)
    mat = oracle.q3_pack(codes)
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    tunable("HQ_Q3_ROW_BLOCKS", 1)
    assert _plan(K, N, M) == PLAN_BLOCK
    y = _run(hq, A, mat, scales, zeros)
    for m in range(M):
        assert rel_err(y[m], exact[m]) <= 1e-3, m
    assert np.array_equal(_run(hq, A, mat, scales, zeros), y)  # partial sums and counters are left ready
    dm, ds, dz = _t(mat), _t(scales), _t(zeros)
    for m in (0, 3, 4, M - 1):
        assert rel_err(y[m], hq.q3_matvec(_t(A[m]), dm, ds, dz).cpu().numpy()) <= 1e-3
    if M <= 12:
        tunable("HQ_Q3_ROW_BLOCKS", 0)
        if _plan(K, N, M) == PLAN_BLOCK:
            # the same digits and the same order of sums within a row: the same bits
            assert np.array_equal(_run(hq, A, mat, scales, zeros), y)


def test_block_kernel_plan_limits(hq, tunable):
    """Beyond 64 rows, beyond four workgroups per compute unit as row blocks (5 and 6 rows: one), for 5 ... 8 rows
    as passes beyond eight rounds of K or where the GEMM's 128-column tiles fill the device, or with more partial
    sums than the fixed scratch of the entry point that allocates nothing holds, the batch takes the GEMM;
    HQ_Q3_SMALL_BATCH lowers the limit.  (The counts below are for 256 compute units.)"""
    assert _plan(32768, 256, 8) == PLAN_BLOCK
    assert _plan(32800, 256, 8) == PLAN_BLOCK         # nine rounds, four tiles: still one workgroup per round, two passes
    assert _plan(49152, 12288, 8) == PLAN_GEMM        # twelve rounds, 192 tiles: six rounds per workgroup, one pass only
    assert _plan(49152, 12288, 4) == PLAN_BLOCK
    assert _plan(4096, 4096, 8) == PLAN_BLOCK
    assert _plan(4096, 4096, 13) == PLAN_BLOCK        # four row blocks: 256 workgroups
    assert _plan(4096, 4096, 32) == PLAN_BLOCK        # eight row blocks: two workgroups per compute unit
    assert _plan(4096, 4096, 64) == PLAN_BLOCK        # sixteen row blocks: four workgroups per compute unit
    assert _plan(4096, 4096, 65) == PLAN_GEMM
    assert _plan(4096, 8192, 64) == PLAN_GEMM         # 128 tiles x 16 row blocks
    assert _plan(4096, 16448, 12) == PLAN_BLOCK       # 257 tiles x 3 row blocks
    assert _plan(4096, 16448, 16) == PLAN_GEMM        # x 4 row blocks: more than four per compute unit
    assert _plan(4096, 16448, 6) == PLAN_BLOCK        # six rows there: two passes of one workgroup per tile
    assert _plan(8192, 8192, 12) == PLAN_BLOCK        # 128 tiles x 2 rounds x 3 row blocks
    assert _plan(8192, 22016, 12) == PLAN_GEMM        # 344 x 2 x 3
    assert _plan(8192, 28672, 4) == PLAN_BLOCK        # one pass per workgroup: always
    assert _plan(8192, 28672, 5) == PLAN_GEMM         # two passes: not where the GEMM's 224 tiles fill the device
    assert _plan(8192, 22016, 8) == PLAN_BLOCK        # 172 tiles of 128 columns: two passes
    assert _plan(28672, 8192, 8) == PLAN_BLOCK
    assert _plan(12288, 65536, 3) == PLAN_BLOCK       # 1024 tiles x 3 rounds x 3 rows would be 9216 partial rows: two ranges of K
    assert _plan(12288, 65536, 8) == PLAN_GEMM        # two passes: one round per workgroup only
    tunable("HQ_Q3_ROW_BLOCKS", 0)                    # passes only: the limits of the passes
    assert _plan(4096, 4096, 12) == PLAN_BLOCK        # three passes: 64 workgroups
    assert _plan(4096, 4096, 13) == PLAN_GEMM
    assert _plan(4096, 16448, 12) == PLAN_GEMM        # 257 workgroups
    assert _plan(8192, 8256, 12) == PLAN_GEMM
    tunable("HQ_Q3_ROW_BLOCKS", -1)
    tunable("HQ_Q3_SMALL_BATCH", 16)
    assert _plan(4096, 4096, 16) == PLAN_BLOCK
    assert _plan(4096, 4096, 17) == PLAN_GEMM
    tunable("HQ_Q3_SMALL_BATCH", 4)
    assert _plan(4096, 4096, 4) == PLAN_BLOCK
    assert _plan(4096, 4096, 5) == PLAN_GEMM
    tunable("HQ_Q3_SMALL_BATCH", 1)
    assert _plan(4096, 4096, 2) == PLAN_GEMM


@pytest.mark.parametrize("scale_exp", [-16, -8, 0, 4])
def test_block_kernel_dynamic_range(hq, oracle, scale_exp):
    """Rows of very different magnitude side by side in one matrix-core operand, an all-zero row, a row with
    one large outlier, magnitudes spread over 2^8 inside a row, a large entry in every k-group, fp16
    subnormals: every row is held to the bound the N(0,1) cases meet, measured against that row's own RMS."""
    K, N = 2048, 2052
    rng = np.random.default_rng(211 + scale_exp)
    codes, scales, zeros, A = oa.make_q3_problem(280 + scale_exp, K, N, x_dtype=np.float16, batch=9)
    mat = oracle.q3_pack(codes)
    A = A.astype(np.float32) * np.float32(2.0 ** scale_exp)
    A[1] *= np.float32(2.0 ** -6)
    A[2] *= np.float32(2.0 ** 5)
    A[4] = 0.0
    A[5, 100] = np.float32(2.0 ** min(15, scale_exp + 12))
    A[6] = rng.standard_normal(K).astype(np.float32) * np.float32(2.0 ** scale_exp) * \
        np.exp2(rng.integers(-8, 1, K)).astype(np.float32)
    A[7, 512:] = 0.0
    A[8, ::32] *= np.float32(64.0)                         # one large entry in every group of 32
    A = A.astype(np.float16)
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    for rows in (list(range(8)), [5, 4, 1, 2], [6, 7, 8], [8, 3, 5, 0, 4, 7]):
        sub = np.ascontiguousarray(A[rows])
        assert _plan(K, N, len(rows)) == PLAN_BLOCK
        y = _run(hq, sub, mat, scales, zeros)
        for i, m in enumerate(rows):
            if m == 4:
                assert np.all(y[i] == 0.0)
            else:
                assert rel_err(y[i], exact[m]) <= 5e-3, (scale_exp, m)
                assert rel_err(y[i], exact[m], FLOOR_F16) <= 1e-4, (scale_exp, m)


def test_block_kernel_non_finite_activations(hq, oracle):
    """An infinity or NaN in one row makes that row NaN and leaves the other rows alone."""
    K, N = 4608, 1024
    codes, scales, zeros, A = oa.make_q3_problem(92, K, N, x_dtype=np.float16, batch=6)
    mat = oracle.q3_pack(codes)
    A[1, 37] = np.float16(np.inf)
    A[4, 4500] = np.float16(np.nan)
    assert _plan(K, N, 6) == PLAN_BLOCK
    y = _run(hq, A, mat, scales, zeros)
    exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
    for m in (0, 2, 3, 5):
        assert rel_err(y[m], exact[m]) <= 5e-3
    assert np.all(np.isnan(y[1])) and np.all(np.isnan(y[4]))


def test_block_kernel_accumulates_and_strict_fences(hq, oracle, tunable):
    import torch
    from hecbench_amd import _lib
    for (M, K, N) in [(5, 12288, 2052), (3, 512, 8196)]:     # K split three ways; one workgroup per tile
        codes, scales, zeros, A = oa.make_q3_problem(433 + M, K, N, x_dtype=np.float16, batch=M)
        mat = oracle.q3_pack(codes)
        y0 = np.random.default_rng(7).standard_normal((M, N)).astype(np.float32)
        dA, dm, ds, dz = _t(A), _t(mat), _t(scales), _t(zeros)
        assert _plan(K, N, M) == PLAN_BLOCK
        plain = _run(hq, A, mat, scales, zeros)
        _check(plain, oracle.q3_gemm(A, mat, scales, zeros, mode=0))
        for strict in (0, 1):
            tunable("HQ_SPLITK_FENCES", strict)
            dy = _t(y0)
            rc = _lib.load().hq_q3_matvec(dA.data_ptr(), 1, dm.data_ptr(), ds.data_ptr(), dz.data_ptr(), dy.data_ptr(),
                                          K, N, M, 1, None)
            assert rc == 0
            torch.cuda.synchronize()
            assert np.array_equal(dy.cpu().numpy(), y0 + plain)   # one fp32 addition to the finished sum


@pytest.mark.parametrize("K", [32, 96, 160])
def test_block_kernel_short_k(hq, oracle, K):
    """Fewer k-groups than a workgroup's waves cover: idle waves, partly filled steps."""
    N = 520
    codes, scales, zeros, A = oa.make_q3_problem(800 + K, K, N, x_dtype=np.float16, batch=7)
    mat = oracle.q3_pack(codes)
    assert _plan(K, N, 7) == PLAN_BLOCK
    _check(_run(hq, A, mat, scales, zeros), oracle.q3_gemm(A, mat, scales, zeros, mode=0))


def test_small_batches_random_shapes(hq, oracle):
    """Twenty seeded shapes: K any multiple of 32 up to 12 rounds, N any multiple of 4, batches 2 ... 8."""
    rng = np.random.default_rng(20250)
    for case in range(20):
        K = 32 * int(rng.integers(1, 1536 if case % 5 == 0 else 300))
        N = 4 * int(rng.integers(1, 700))
        M = int(rng.integers(2, 9))
        codes, scales, zeros, A = oa.make_q3_problem(3000 + case, K, N, x_dtype=np.float16, batch=M)
        mat = oracle.q3_pack(codes)
        if _plan(K, N, M) != PLAN_BLOCK:
            continue
        y = _run(hq, A, mat, scales, zeros)
        exact = oracle.q3_gemm(A, mat, scales, zeros, mode=0)
        for m in range(M):
            assert rel_err(y[m], exact[m]) <= 5e-3, (case, K, N, M, m)
            assert rel_err(y[m], exact[m], FLOOR_F16) <= 1e-4, (case, K, N, M, m)
