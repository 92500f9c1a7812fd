"""hq_reserve_workspace promises that calls up to (max_K, max_N) never allocate: its bound (hq_reserve_need) must
cover the workspace need of every smaller call (hq_q3_workspace_need, computed by the launch's own plan
functions).  Host arithmetic only - no GPU."""
import ctypes
import random

import pytest

from hecbench_amd import _lib


def _need(lib, cus, K, N, M):
    f, c = ctypes.c_int64(), ctypes.c_int64()
    rc = lib.hq_q3_workspace_need(cus, K, N, M, ctypes.byref(f), ctypes.byref(c))
    assert rc == 0, (rc, cus, K, N, M)
    return f.value, c.value


def _bound(lib, cus, K, N):
    f, c = ctypes.c_int64(), ctypes.c_int64()
    assert lib.hq_reserve_need(cus, K, N, ctypes.byref(f), ctypes.byref(c)) == 0
    return f.value, c.value


BATCHES = (1, 2, 3, 4, 5, 6, 7, 8, 9, 12, 13, 16, 24, 32, 33, 48, 64, 65, 72, 128)


@pytest.mark.parametrize("cus", [256, 304, 120, 64])
@pytest.mark.parametrize("max_K,max_N", [(8192, 28672), (16384, 65536), (4096, 4096), (49152, 12288), (1024, 256),
                                         (32768, 1024), (65536, 4096)])
def test_reserve_covers_every_smaller_call(cus, max_K, max_N):
    lib = _lib.load()
    bf, bc = _bound(lib, cus, max_K, max_N)
    rng = random.Random(cus * 1000003 + max_K * 31 + max_N)
    Ks = {max_K, 32, 4096, 8192, 2048, 1024, 128, 14336, 11008, 16384, 28672, 36864, 40960} | \
         {rng.randrange(1, max_K // 32 + 1) * 32 for _ in range(12)}
    Ns = {max_N, 4, 64, 128, 256, 1024, 2048, 4096, 4100, 8192, 11008, 12288, 22016} | \
         {rng.randrange(1, max_N // 4 + 1) * 4 for _ in range(12)}
    worst = (0, (0, 0, 0))
    for K in sorted(k for k in Ks if k <= max_K):
        for N in sorted(n for n in Ns if n <= max_N):
            for M in BATCHES:
                f, c = _need(lib, cus, K, N, M)
                assert f <= bf, ("floats", cus, K, N, M, f, bf)
                assert c <= bc, ("counters", cus, K, N, M, c, bc)
                worst = max(worst, (f, (K, N, M)))
    assert worst[0] > 0 or max_K < 2048


def test_the_case_that_used_to_fall_short():
    # 256 compute units: a reservation for (8192, 28672) must hold M=72, K=8192, N=4096, whose 32 column tiles
    # split K eight ways (re-ordered activations 262,144 floats + 128 + 32 x 8 x 64 x 128 raw sums)
    lib = _lib.load()
    f, _ = _need(lib, 256, 8192, 4096, 72)
    assert f == 262144 + 128 + 32 * 8 * 64 * 128
    bf, _ = _bound(lib, 256, 8192, 28672)
    assert bf >= f
    f2, _ = _need(lib, 256, 16384, 2048, 72)
    assert _bound(lib, 256, 16384, 65536)[0] >= f2


def test_bad_arguments():
    lib = _lib.load()
    f, c = ctypes.c_int64(), ctypes.c_int64()
    assert lib.hq_q3_workspace_need(256, 100, 64, 1, ctypes.byref(f), ctypes.byref(c)) < 0
    assert lib.hq_q3_workspace_need(0, 128, 64, 1, ctypes.byref(f), ctypes.byref(c)) < 0
    assert lib.hq_reserve_need(256, -1, 64, ctypes.byref(f), ctypes.byref(c)) < 0
    assert lib.hq_reserve_need(256, 128, 64, None, ctypes.byref(c)) < 0
