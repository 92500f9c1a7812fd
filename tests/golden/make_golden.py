"""Writes the golden fixtures of this folder from the REFERENCE compiled out of its own
sources (oracle/_ref, built by `make -C oracle ref` where the HeCBench tree is mounted).
The fixtures are data only: inputs and the outputs the reference's own host loops produce.

    python tests/golden/make_golden.py
"""
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from tests import oracle_api as oa  # noqa: E402


def lut_fixture(ref, name, N, K, NB):
    """src/lut-gemm-hip/main.cu:101-146: rand()-seeded bit planes, alphas, biases and the
    dense weights dequantizeFrom_qW() derives from them (weight[n*K + k])."""
    G = K // 128
    qW = np.zeros((K, NB, N), np.float32)
    bW = np.zeros((K // 32, NB, N), np.uint32)
    alpha = np.zeros((G, NB, N), np.float32)
    qbias = np.zeros((G, N), np.float32)
    weight = np.zeros((N, K), np.float32)
    inp = np.zeros(K, np.float32)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    getattr(ref, name)(vp(qW), vp(bW), vp(alpha), vp(qbias), vp(weight), vp(inp))
    np.savez_compressed(os.path.join(HERE, f"lut_fixture_{N}x{K}x{NB}.npz"), signs=qW.astype(np.int8), bW=bW,
                        alpha=alpha, q_bias=qbias, weight=weight, input=inp)


def dquantize_fixture(ref_cpu):
    """src/quantBnB-omp/main.cpp: the host quantiser on a fixed input vector, with the table
    reduced to what a checker needs: the 256 fp32 values the function searched."""
    rng = np.random.default_rng(19937)
    A = np.concatenate([rng.standard_normal(8192).astype(np.float32),
                        np.linspace(-1.2, 1.2, 4096, dtype=np.float32)])
    out = np.zeros(A.size, np.uint8)
    ref_cpu.ref_dquantize_n(A.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p),
                            ctypes.c_long(A.size))
    np.savez_compressed(os.path.join(HERE, "dquantize_outputs.npz"), A=A, out=out)


def main():
    ref = oa.load_ref_hip()
    ref_cpu = oa.load_ref_cpu()
    assert ref is not None and ref_cpu is not None, "build oracle/_ref first: make -C oracle ref"
    lut_fixture(ref, "ref_lut_fixture_256x256x3", 256, 256, 3)
    dquantize_fixture(ref_cpu)


if __name__ == "__main__":
    main()
