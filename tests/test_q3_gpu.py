"""Parity of hq_q3_matvec (batch 1) with the CPU oracle, through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import FLOOR_F16, TOL_F16_ACC, TOL_F32_ACC, rel_err

pytestmark = pytest.mark.gpu


def _run(hq, x, mat, scales, zeros, out=None, accumulate=False):
    import torch
    dev = torch.device("cuda:0")
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    o = None if out is None else t(out)
    y = hq.q3_matvec(t(x), t(mat), t(scales), t(zeros), out=o, accumulate=accumulate)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def _reference_pattern(K, N):
    """Weights of the reference's own check: every code is 1 (main.cu:35-43)."""
    p1 = 0b01001001001001001001001001001001
    mat = np.zeros((3 * K // 32, N), np.uint32)
    mat[0::3] = p1
    mat[1::3] = (p1 << 1) & 0xFFFFFFFF
    mat[2::3] = (p1 << 2) & 0xFFFFFFFF
    return mat.view(np.int32)


def test_known_answer_minus_49152(hq):
    """The reference's verification: x=1, scale=-1, zero=0, all codes 1, K=49152 ->
    every output is exactly -49152 (src/quant3MatMul-hip/main.cu:84-105), fp32 and fp16 input."""
    K, N = 49152, 12288
    mat = _reference_pattern(K, N)
    s = -np.ones(N, np.float32)
    z = np.zeros(N, np.float32)
    y = _run(hq, np.ones(K, np.float32), mat, s, z)
    assert (y == -49152.0).all()
    y = _run(hq, np.ones(K, np.float16), mat, s, z)
    assert (y == -49152.0).all()
    # the reference wrappers accumulate into mul: start from 1000 -> -48152
    y = _run(hq, np.ones(K, np.float32), mat, s, z, out=np.full(N, 1000, np.float32), accumulate=True)
    assert (y == -48152.0).all()


@pytest.mark.parametrize("K,N,seed", [(4096, 11008, 11), (256, 256, 12), (1024, 64, 13), (32, 4, 14),
                                      (4096, 1000, 15), (8192, 4096, 16), (6144, 320, 17), (160, 132, 18)])
def test_matvec_f32_vs_oracle(hq, oracle, K, N, seed):
    codes, scales, zeros, x = oa.make_q3_problem(seed, K, N)
    mat = oracle.q3_pack(codes)
    y = _run(hq, x, mat, scales, zeros)
    ref64 = oracle.q3_matvec_f64(x, mat, scales, zeros)
    ref32 = oracle.q3_matvec_f32(x, mat, scales, zeros)
    assert rel_err(y, ref32) <= TOL_F32_ACC
    # fp32-accumulate accuracy: as close to the exact sum as the reference's own fp32 order
    assert rel_err(y, ref64) <= 1e-4


@pytest.mark.parametrize("K,N,seed", [(4096, 11008, 21), (512, 256, 22), (32, 4, 23), (160, 132, 24), (8192, 512, 25)])
def test_matvec_f16_vs_oracle(hq, oracle, K, N, seed):
    codes, scales, zeros, x = oa.make_q3_problem(seed, K, N, x_dtype=np.float16)
    mat = oracle.q3_pack(codes)
    y = _run(hq, x, mat, scales, zeros)
    ref16 = oracle.q3_matvec_f16(x, mat, scales, zeros)          # the reference's fp16 arithmetic
    ref64 = oracle.q3_matvec_f64(x.astype(np.float64), mat, scales, zeros)
    assert rel_err(y, ref16, FLOOR_F16) <= TOL_F16_ACC
    assert rel_err(y, ref64) <= 1e-4   # fp32 accumulation: far tighter than the fp16 contract


def test_integer_exact(hq, oracle):
    """scale=1, zero=0, small integer x: the result is an exact integer matvec."""
    K, N = 2048, 512
    rng = np.random.default_rng(5)
    codes = rng.integers(0, 8, size=(K, N), dtype=np.uint8)
    x = rng.integers(-8, 9, size=K).astype(np.float32)
    mat = oracle.q3_pack(codes)
    y = _run(hq, x, mat, np.ones(N, np.float32), np.zeros(N, np.float32))
    want = x.astype(np.int64) @ codes.astype(np.int64)
    assert (y.astype(np.int64) == want).all() and (y == np.round(y)).all()


def test_each_code_position(hq, oracle):
    """One non-zero code at every position of a k-group: catches a wrong field
    mask, a wrong power-of-two slot scale or a swapped activation slot."""
    K, N = 64, 64
    for k in range(K):
        codes = np.zeros((K, N), np.uint8)
        codes[k, :] = np.arange(N) % 8
        x = np.zeros(K, np.float32)
        x[k] = 1.0 + k / 64.0
        x[(k + 1) % K] = 100.0  # must not leak in
        mat = oracle.q3_pack(codes)
        y = _run(hq, x, mat, np.ones(N, np.float32), np.zeros(N, np.float32))
        assert np.array_equal(y, (np.arange(N) % 8) * np.float32(1.0 + k / 64.0)), k


def test_wide_dynamic_range_and_zero_vector(hq, oracle):
    K, N = 1024, 256
    codes, scales, zeros, x = oa.make_q3_problem(31, K, N)
    mat = oracle.q3_pack(codes)
    for scale in (1e-30, 1e-6, 1e6, 1e30):
        xs = (x * np.float32(scale)).astype(np.float32)
        y = _run(hq, xs, mat, scales, zeros)
        ref = oracle.q3_matvec_f64(xs, mat, scales, zeros)
        assert rel_err(y, ref) <= 1e-4, scale
    y = _run(hq, np.zeros(K, np.float32), mat, scales, zeros)
    assert (y == 0).all()


def test_non_finite_activations_propagate(hq, oracle):
    K, N = 512, 128
    codes, scales, zeros, x = oa.make_q3_problem(33, K, N)
    mat = oracle.q3_pack(codes)
    for bad in (np.nan, np.inf, -np.inf):
        xs = x.copy()
        xs[77] = bad
        for z in (zeros, np.zeros_like(zeros)):
            y = _run(hq, xs, mat, scales, z)
            assert not np.isfinite(y).any(), bad


def test_launch_shapes_match(hq, oracle, tunable):
    """Every launch shape (waves per workgroup x steps x K split; one or several
    rounds per workgroup) gives the same answer."""
    K, N = 4096, 1024
    codes, scales, zeros, x = oa.make_q3_problem(41, K, N)
    mat = oracle.q3_pack(codes)
    ref = oracle.q3_matvec_f64(x, mat, scales, zeros)
    for waves, steps, ks in [(8, 4, 0), (8, 2, 0), (4, 2, 1), (4, 1, 0), (16, 1, 1), (8, 4, 1), (4, 4, 2), (4, 8, 0),
                             (8, 1, 3), (8, 1, 1), (4, 1, 1)]:
        tunable("HQ_Q3_WAVES", waves)
        tunable("HQ_Q3_STEPS", steps)
        tunable("HQ_Q3_KSPLIT", ks)
        for _ in range(2):  # twice: the arrival counters must reset themselves
            y = _run(hq, x, mat, scales, zeros)
            assert rel_err(y, ref) <= 1e-4, (waves, steps, ks)
            if ks > 1:  # formal release/acquire fences in the split-K arrival: the same bits
                tunable("HQ_SPLITK_FENCES", 1)
                assert np.array_equal(_run(hq, x, mat, scales, zeros), y), (waves, steps, ks)
                tunable("HQ_SPLITK_FENCES", 0)


@pytest.mark.parametrize("x_dtype", [np.float32, np.float16])
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 1028), (160, 132), (32, 4), (8192, 1024), (12320, 516), (4096, 11008),
                                 (32768, 68)])
def test_narrow_tiles_match(hq, oracle, tunable, K, N, x_dtype):
    """Tiles of 32 and 16 columns (chosen by default where 64-column tiles would leave more than half of the
    compute units without a workgroup) against the 64-column tiles, forced on shapes with ragged last tiles,
    K splits and many tiles: the same bits (a column's arithmetic does not depend on its tile), accumulation
    included, and the oracle's result."""
    codes, scales, zeros, x = oa.make_q3_problem(K + N, K, N, x_dtype=x_dtype)
    mat = oracle.q3_pack(codes)
    exact = oracle.q3_matvec_f64(x, mat, scales, zeros)
    y0 = np.linspace(-1.0, 1.0, N).astype(np.float32)
    tunable("HQ_Q3_TILE", 4)
    wide = _run(hq, x, mat, scales, zeros)
    wide_acc = _run(hq, x, mat, scales, zeros, out=y0.copy(), accumulate=True)
    assert rel_err(wide, exact, FLOOR_F16) <= 1e-3
    for cpl in (2, 1):
        tunable("HQ_Q3_TILE", cpl)
        assert np.array_equal(_run(hq, x, mat, scales, zeros), wide), cpl
        assert np.array_equal(_run(hq, x, mat, scales, zeros, out=y0.copy(), accumulate=True), wide_acc), cpl
        assert np.array_equal(_run(hq, x, mat, scales, zeros), wide), cpl  # counters left ready


@pytest.mark.parametrize("K,N", [(8192, 22016), (16384, 16644), (28672, 1028), (5120, 13824)])
def test_default_k_split_on_long_k(hq, oracle, tunable, K, N):
    """Up to eight rounds of K run as one workgroup per round whatever the tile count (more column tiles than
    compute units included): sampled columns against the oracle, every column against the unsplit launch."""
    rng = np.random.default_rng(K + N)
    mat = rng.integers(-2 ** 31, 2 ** 31, size=(3 * K // 32, N), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, size=N).astype(np.float32)
    zeros = (scales * rng.integers(3, 5, size=N)).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    y = _run(hq, x, mat, scales, zeros)
    y_again = _run(hq, x, mat, scales, zeros)          # the arrival counters reset themselves
    assert np.array_equal(y, y_again)
    cols = np.unique(np.concatenate([np.arange(0, 68), np.arange(N - 68, N), rng.integers(0, N, 64)]))
    ref = oracle.q3_matvec_f64(x, np.ascontiguousarray(mat[:, cols]), scales[cols], zeros[cols])
    assert rel_err(y[cols], ref) <= 1e-4
    tunable("HQ_Q3_KSPLIT", 1)
    assert rel_err(y, _run(hq, x, mat, scales, zeros)) <= 1e-4


@pytest.mark.parametrize("K,N,x_dtype", [(36864, 16384, np.float32), (33792, 16388, np.float16), (36864, 4096, np.float32)])
def test_more_than_eight_rounds_of_k(hq, oracle, tunable, K, N, x_dtype):
    """More than eight rounds of K.  256 tiles fill the compute units evenly: unsplit workgroups walk the
    rounds, the next round's loads going out a step at a time.  257 tiles (the last one 4 columns wide, a K the
    rounds do not divide) and 64 tiles do not: one workgroup per round, nine partial sums per tile, added up
    in two batches of loads.  Sampled columns against the oracle, every column against a three-way split whose
    workgroups walk several rounds, the same bits on a second call."""
    rng = np.random.default_rng(K + N)
    mat = rng.integers(-2 ** 31, 2 ** 31, size=(3 * K // 32, N), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, size=N).astype(np.float32)
    zeros = (scales * rng.integers(3, 5, size=N)).astype(np.float32)
    x = rng.standard_normal(K).astype(x_dtype)
    y = _run(hq, x, mat, scales, zeros)
    assert np.array_equal(y, _run(hq, x, mat, scales, zeros))
    cols = np.unique(np.concatenate([np.arange(0, 68), np.arange(N - 68, N), rng.integers(0, N, 64)]))
    ref = oracle.q3_matvec_f64(x.astype(np.float32), np.ascontiguousarray(mat[:, cols]), scales[cols], zeros[cols])
    assert rel_err(y[cols], ref) <= 1e-4
    tunable("HQ_Q3_KSPLIT", 3)
    assert rel_err(y, _run(hq, x, mat, scales, zeros)) <= 2e-4   # two results, each within 1e-4 of the exact one


def test_rejects_bad_arguments(hq):
    import torch
    dev = torch.device("cuda:0")
    x = torch.zeros(64, device=dev)
    w = torch.zeros((6, 8), dtype=torch.int32, device=dev)
    s = torch.zeros(8, device=dev)
    with pytest.raises(hq.HqError):
        hq.q3_matvec(x, torch.zeros((6, 6), dtype=torch.int32, device=dev), s[:6], s[:6])  # N % 4
    with pytest.raises(ValueError):
        hq.q3_matvec(x, w[:3], s, s)  # wrong packed height
    with pytest.raises(ValueError):
        hq.q3_matvec(x.cpu(), w, s, s)  # no CPU path


def test_vs_reference_kernels(hq, oracle):
    """Where the reference's own HIP kernels were compiled into oracle/_ref, run
    them on the same device buffers: fp32 kernel and fp16 'faster' kernel."""
    import torch
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built")
    dev = torch.device("cuda:0")
    K, N = 4096, 11008  # both multiples of 256, as the reference grid requires
    codes, scales, zeros, x = oa.make_q3_problem(51, K, N)
    mat = oracle.q3_pack(codes)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    dx, dm, ds, dz = t(x), t(mat), t(scales), t(zeros)
    dx16 = t(x.astype(np.float16))
    vp = lambda a: ctypes.c_void_p(a.data_ptr())
    mul = torch.zeros(N, device=dev)
    ref.ref_vecquant3matmul_f32(vp(dx), vp(dm), vp(mul), vp(ds), vp(dz), 3 * K // 32, N)
    torch.cuda.synchronize()
    y = hq.q3_matvec(dx, dm, ds, dz)
    torch.cuda.synchronize()
    assert rel_err(y.cpu().numpy(), mul.cpu().numpy()) <= TOL_F32_ACC
    mul16 = torch.zeros(N, device=dev)
    ref.ref_vecquant3matmul_faster(vp(dx16), vp(dm), vp(mul16), vp(ds), vp(dz), 3 * K // 32, N)
    torch.cuda.synchronize()
    y16 = hq.q3_matvec(dx16, dm, ds, dz)
    torch.cuda.synchronize()
    assert rel_err(y16.cpu().numpy(), mul16.cpu().numpy(), FLOOR_F16) <= TOL_F16_ACC
    # and the oracle's restatement of the fp16 kernel agrees with the real one
    o16 = oracle.q3_matvec_f16(x.astype(np.float16), mat, scales, zeros)
    assert rel_err(o16, mul16.cpu().numpy(), FLOOR_F16) <= 2e-3
