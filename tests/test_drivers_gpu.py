"""The benchmark drivers keep the reference command lines and verification contracts: run each
one with a small problem and check its verdict."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BENCH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "hecbench_amd", "bench")

CASES = [
    (["quant3MatMul", "3"], ["PASS", "Average execution time of the kernel:", "Average execution time of the faster kernel:"]),
    (["quantBnB", "1048576", "2"], ["PASS", "Average execution time of kQuantize kernel with block size"]),
    (["lut-gemm", "1", "2"], ["M = 1, N = ", "LUT-GEMM [INT3, FP16, FP16]", "mean Error:", "latency min :"]),
    (["quantAQLM"], ["kernel execution time:"]),
    (["quantVLLM", "64", "512", "2"], ["Input type is FP16", "Input type is BF16", "Input type is FP32", "PASS"]),
    (["gemv", "-s", "512", "-i", "2"], ["GEMV FP16 ..", "GEMV int8 quantized...", "GEMV int4 quantized...", "PASS"]),
    (["mxfp4", "65536", "2"], ["Bandwidth (GB/sec):", "PASS"]),
]


@pytest.mark.parametrize("argv,expect", CASES, ids=[c[0][0] for c in CASES])
def test_driver(argv, expect):
    exe = os.path.join(BENCH, argv[0])
    if not os.path.exists(exe):
        pytest.skip(f"{argv[0]} is not built (run the build step)")
    r = subprocess.run([exe] + argv[1:], capture_output=True, text=True, timeout=100)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out[-2000:]
    assert "FAIL" not in out, out[-2000:]
    for needle in expect:
        assert needle in out, (needle, out[-2000:])
