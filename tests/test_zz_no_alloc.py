"""hq_q3_matvec_noalloc, the entry point that allocates nothing: through the C ABI, bit-identical with
hq_q3_matvec (same kernels, scratch in a fixed device array instead of the stream's workspace) on two
calls in a row, the second with a smaller input, for the split-K matvec and for the batched path."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import rel_err

pytestmark = pytest.mark.gpu


def _problem(oracle, seed, K, N, M):
    import torch
    dev = torch.device("cuda:0")
    codes, scales, zeros, x = oa.make_q3_problem(seed, K, N)
    mat = oracle.q3_pack(codes)
    A = np.random.default_rng(seed).standard_normal((M, K)).astype(np.float16)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    return dict(K=K, N=N, M=M, x=t(x), mat=t(mat), s=t(scales), z=t(zeros), A=t(A),
                host=(x, mat, scales, zeros, A))


def _call(fn, p, batch):
    import torch
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    act = p["A"] if batch > 1 else p["x"]
    y = torch.full((batch, p["N"]), float("nan"), device="cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = fn(vp(act), 1 if batch > 1 else 0, vp(p["mat"]), vp(p["s"]), vp(p["z"]), vp(y), p["K"], p["N"], batch, 0, stream)
    assert rc == 0, rc
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_noalloc_matches_workspace_path(hq, oracle):
    from hecbench_amd import _lib
    lib = _lib.load()
    # 32 and 8 column tiles: far fewer than half the compute units, so both calls split K across
    # workgroups and use the partial sums and the arrival counters
    big = _problem(oracle, 301, 8192, 2048, 70)
    small = _problem(oracle, 302, 2048, 512, 66)
    for p in (big, small):                      # two calls in a row, the second with a smaller input
        # the matvec (narrow tiles), the small-batch kernel with one workgroup per tile and with two, three and
        # ten row blocks, the GEMM (64 rows and the rest)
        for batch in (1, 2, 6, 11, 40, p["M"]):
            want = _call(lib.hq_q3_matvec, p, batch)
            got = _call(lib.hq_q3_matvec_noalloc, p, batch)
            assert np.array_equal(got, want), (p["K"], p["N"], batch)
            x, mat, scales, zeros, A = p["host"]
            if batch == 1:
                assert rel_err(got[0], oracle.q3_matvec_f64(x, mat, scales, zeros)) <= 1e-4
            else:
                assert rel_err(got, oracle.q3_gemm(A[:batch], mat, scales, zeros, mode=0)) <= 5e-3
    # and again in the other order: the array keeps the last call's contents
    for p in (small, big, small):
        assert np.array_equal(_call(lib.hq_q3_matvec_noalloc, p, 1), _call(lib.hq_q3_matvec, p, 1))


def test_noalloc_rejects_beyond_its_limits(hq):
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    K, N, M = 32768, 64, 65                     # the batched GEMM's activations would need 4 MiB
    A = torch.zeros((M, K), dtype=torch.float16, device=dev)
    w = torch.zeros((3 * K // 32, N), dtype=torch.int32, device=dev)
    s = torch.zeros(N, device=dev)
    y = torch.zeros((M, N), device=dev)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    assert lib.hq_q3_matvec_noalloc(vp(A), 1, vp(w), vp(s), vp(s), vp(y), K, N, M, 0, None) == -6
    assert lib.hq_q3_matvec(vp(A), 1, vp(w), vp(s), vp(s), vp(y), K, N, M, 0, None) == 0
    torch.cuda.synchronize()
    assert lib.hq_q3_matvec_noalloc(None, 0, None, None, None, None, 64, 8, 1, 0, None) == -1
