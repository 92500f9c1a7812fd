"""CPU legs of the benchmark report: the oracle's loops spread over threads give the serial results, and the
quantBnB driver's host-only mode (its own verification loops under OpenMP, no GPU call) keeps the benchmark's
printed contract."""
import os
import subprocess

import numpy as np
import pytest

from tests import oracle_api as oa

BENCH = os.path.join(oa.ROOT, "hecbench_amd", "bench")


@pytest.fixture(scope="module")
def o():
    return oa.load_oracle()


def test_threaded_oracle_equals_serial(o):
    packed, absmax = oa.make_nf4_problem(3, 64 * 1000, 64)
    bW, alpha, qb, x = oa.make_lut_problem(3, 512, 192, 3, 128)
    codes, cb, sc, xa = oa.make_aqlm_problem(3, 96, 256)
    qc, scales, zeros, A = oa.make_q3_problem(3, 256, 128, np.float16, batch=3)
    mat = o.q3_pack(qc)
    jobs = [lambda: o.dequant_4bit(packed, absmax, 64 * 1000, 64),
            lambda: o.lut_gemv_f64(bW, alpha, qb, x, 128),
            lambda: o.aqlm_matvec(codes, cb, sc, xa, (96, 0, 0, 0), 65536),
            lambda: o.q3_gemm(A, mat, scales, zeros)]
    try:
        for job in jobs:
            o.set_threads(1)
            want = job()
            o.set_threads(4)
            got = job()
            want = want if isinstance(want, tuple) else (want,)
            got = got if isinstance(got, tuple) else (got,)
            for a, b in zip(want, got):
                assert np.array_equal(np.asarray(a), np.asarray(b))
    finally:
        o.set_threads(1)


def test_quantbnb_host_only_mode_needs_no_gpu():
    exe = os.path.join(BENCH, "quantBnB")
    if not os.path.exists(exe):
        pytest.skip("quantBnB is not built (run the build step)")
    env = dict(os.environ, OMP_NUM_THREADS="4", HIP_VISIBLE_DEVICES="")
    r = subprocess.run([exe, "131072", "2", "--host-only"], capture_output=True, text=True, timeout=100, env=env)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out[-2000:]
    assert "FAIL" not in out
    assert out.count("PASS") == 2
    assert "Average execution time of kQuantize kernel with block size 256:" in out
    assert "host only: OpenMP loop on 4 threads" in out
    r = subprocess.run([exe, "131072"], capture_output=True, text=True, timeout=100, env=env)
    assert r.returncode == 1 and "Usage:" in r.stdout
