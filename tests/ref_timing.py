"""Manual measurement (not collected by pytest): times the REFERENCE's own HIP kernels,
compiled from the reference tree into oracle/_ref/libhecref_hip.so, next to libhq on
the same device buffers.  Run on a GPU box:  python tests/ref_timing.py"""
import ctypes
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import hecbench_amd as hq  # noqa: E402
from tests import oracle_api as oa  # noqa: E402


def timeit(fn, iters, warmup=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def main():
    ref = oa.load_ref_hip()
    assert ref is not None, "oracle/_ref/libhecref_hip.so not built"
    dev = torch.device("cuda:0")
    hq.init()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    g = torch.Generator(device=dev)
    g.manual_seed(5)
    for K, N in ((4096, 11008), (49152, 12288)):
        rows = 3 * K // 32
        nbuf = max(2, int(600e6 // (rows * N * 4)) + 1)
        mats = [torch.randint(-2 ** 31, 2 ** 31 - 1, (rows, N), dtype=torch.int32, device=dev, generator=g)
                for _ in range(nbuf)]
        s = torch.empty(N, device=dev).uniform_(0.005, 0.02, generator=g)
        z = s * 3
        x = torch.randn(K, device=dev, generator=g)
        x16 = x.half()
        y = torch.zeros(N, device=dev)
        it = [0]

        def ref32():
            y.zero_()  # the reference caller memsets before each launch
            ref.ref_vecquant3matmul_f32(vp(x), vp(mats[it[0] % nbuf]), vp(y), vp(s), vp(z), rows, N)
            it[0] += 1

        def ref16():
            y.zero_()
            ref.ref_vecquant3matmul_faster(vp(x16), vp(mats[it[0] % nbuf]), vp(y), vp(s), vp(z), rows, N)
            it[0] += 1

        def ours():
            hq.q3_matvec(x, mats[it[0] % nbuf], s, z, out=y)
            it[0] += 1

        n = 300 if K > 8192 else 2000
        print(f"q3 matvec K={K} N={N}: reference fp32 kernel {timeit(ref32, n):.2f} us, reference 'faster' kernel "
              f"{timeit(ref16, n):.2f} us (both incl. their memset), libhq {timeit(ours, n):.2f} us")
    # LUT-GEMM, reference problem shape of `lut-gemm 1 <repeat>` third fixture
    K, N, nb, G = 4096, 16384, 3, 128
    bW = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // 32, nb, N), dtype=torch.int32, device=dev, generator=g)
    al = (torch.randn(K // G, nb, N, device=dev, generator=g) * 0.02).abs().half()
    qb = torch.zeros(K // G, N, dtype=torch.float16, device=dev)
    x16 = torch.randn(K, device=dev, generator=g).half()
    y16 = torch.zeros(N, dtype=torch.float16, device=dev)
    print(f"LUT-GEMM K={K} N={N} q=3 (hot cache): reference matmul() "
          f"{timeit(lambda: ref.ref_lut_matmul(vp(y16), vp(x16), vp(bW), vp(al), vp(qb), K, N, nb, K // G), 300):.2f} us, "
          f"libhq {timeit(lambda: hq.lut_matmul(x16, bW, al, qb, G, out=y16), 300):.2f} us")
    # AQLM, reference problem
    M, K = 12288, 4096
    codes = torch.randint(-32768, 32768, (M, K // 8), dtype=torch.int16, device=dev, generator=g)
    cb = (torch.randn(3, 65536, 8, device=dev, generator=g) * 0.05).half()
    xa = torch.randn(K, device=dev, generator=g).half()
    ya = torch.zeros(M, dtype=torch.float16, device=dev)
    sizes = (ctypes.c_int * 4)(4096, 8192, 12288, 122880)
    print(f"AQLM M={M} K={K} (hot cache): reference kernel "
          f"{timeit(lambda: ref.ref_code1x16_launch(vp(codes), vp(xa), vp(ya), vp(cb), M, K, sizes, 65536, None), 300):.2f} us, "
          f"libhq {timeit(lambda: hq.code1x16_matvec(codes, xa, cb, (4096, 8192, 12288, 122880), 65536, out=ya), 300):.2f} us")
    # kQuantize
    n = 16777216
    ref.ref_hip_code_table.restype = ctypes.POINTER(ctypes.c_float)
    code = torch.from_numpy(np.ctypeslib.as_array(ref.ref_hip_code_table(), shape=(256,)).copy()).to(dev)
    A = torch.randn(n, device=dev, generator=g)
    out = torch.zeros(n, dtype=torch.uint8, device=dev)
    print(f"kQuantize n={n}: reference kernel "
          f"{timeit(lambda: ref.ref_kquantize(vp(code), vp(A), vp(out), ctypes.c_long(n), None), 50):.2f} us, "
          f"libhq {timeit(lambda: hq.quantize_dynamic8(code, A, out=out), 50):.2f} us")


if __name__ == "__main__":
    main()
