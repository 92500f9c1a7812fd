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

        lib = hq._lib.load()  # raw C-ABI calls with prepared arguments: a Python wrapper would cost more
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)  # than these kernels take
        pm = [vp(m) for m in mats]
        px, ps, pz, py = vp(x), vp(s), vp(z), vp(y)

        def ours():
            lib.hq_q3_matvec(px, 0, pm[it[0] % nbuf], ps, pz, py, K, N, 1, 0, stream)
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
          f"libhq {timeit(lambda: lib.hq_lut_gemv(vp(bW), vp(al), vp(qb), vp(x16), vp(y16), K, N, nb, G, stream), 300):.2f} us")
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
    # gemv at the reference's run size and launch shape (src/gemv-hip/Makefile:55)
    n = 16384
    vec = torch.rand(n, device=dev, generator=g).half()
    res = torch.zeros(n, dtype=torch.float16, device=dev)
    cu, cf = ctypes.c_uint, ctypes.c_float
    m16 = torch.rand(n, n, device=dev, generator=g).half()
    print(f"gemv fp16 {n}: reference kernel (512,2) "
          f"{timeit(lambda: ref.ref_gemv_fp16(vp(m16), vp(vec), vp(res), cu(n), cu(512), cu(2), None), 50):.1f} us, "
          f"libhq {timeit(lambda: hq.gemv_fp16(m16, vec, out=res), 50):.1f} us")
    del m16
    m8 = torch.randint(-128, 128, (n, n), dtype=torch.int8, device=dev, generator=g)
    print(f"gemv int8 {n}: reference kernel (512,2) "
          f"{timeit(lambda: ref.ref_gemv_int8(vp(m8), vp(vec), vp(res), cu(n), cf(0.0625), cf(0.01), cu(512), cu(2), None), 50):.1f} us, "
          f"libhq {timeit(lambda: hq.gemv_int8(m8, vec, 0.0625, 0.01, out=res), 50):.1f} us")
    del m8
    m4 = torch.randint(0, 256, (n, n // 2), dtype=torch.uint8, device=dev, generator=g)
    print(f"gemv int4 {n}: reference kernel (512,2) "
          f"{timeit(lambda: ref.ref_gemv_int4(vp(m4), vp(vec), vp(res), cu(n), cf(0.0625), cf(0.01), cu(512), cu(2), None), 50):.1f} us, "
          f"libhq {timeit(lambda: hq.gemv_int4(m4, vec, 0.0625, 0.01, out=res), 50):.1f} us")
    del m4
    # mxfp4 quantise-dequantise, 2^28 fp16 elements (beyond the Infinity Cache)
    nel = 1 << 28
    src = torch.randn(nel, device=dev, generator=g).half()
    dst = torch.empty_like(src)
    print(f"mxfp4 fp16 n={nel}: reference kernel "
          f"{timeit(lambda: ref.ref_mxfp4_qdq(vp(src), vp(dst), ctypes.c_int(nel), ctypes.c_int(0), None), 20):.1f} us, "
          f"libhq {timeit(lambda: hq.mxfp4_qdq(src, out=dst), 20):.1f} us")
    del src, dst
    # quantVLLM at the reference's run size (4096 tokens of 5137 fp16), inputs rotated over 12 tensors
    if hasattr(ref, "ref_hip_int8_quant_static"):
        tk, hd = 4096, 5137
        xs = [torch.randint(-300, 700, (tk, hd), device=dev, generator=g).half() for _ in range(12)]
        q = torch.empty(tk, hd, dtype=torch.int8, device=dev)
        sc = torch.empty(tk, device=dev)
        zp = torch.empty(tk, dtype=torch.int32, device=dev)
        lib = hq._lib.load()
        it = [0]

        def nxt():
            it[0] += 1
            return xs[it[0] % len(xs)]
        cl = ctypes.c_long
        for name, rf, of in (
                ("static", lambda: ref.ref_hip_int8_quant_static(vp(nxt()), 1, vp(q), cl(tk), hd, cf(0.1), 0),
                 lambda: lib.hq_int8_quant_static(vp(nxt()), 1, vp(q), tk, hd, 0.1, 0, 0, None)),
                ("static azp", lambda: ref.ref_hip_int8_quant_static(vp(nxt()), 1, vp(q), cl(tk), hd, cf(0.1), 54),
                 lambda: lib.hq_int8_quant_static(vp(nxt()), 1, vp(q), tk, hd, 0.1, 1, 54, None)),
                ("dynamic", lambda: ref.ref_hip_int8_quant_dynamic(vp(nxt()), 1, vp(q), vp(sc), None, cl(tk), hd),
                 lambda: lib.hq_int8_quant_dynamic(vp(nxt()), 1, vp(q), vp(sc), None, tk, hd, None)),
                ("dynamic azp", lambda: ref.ref_hip_int8_quant_dynamic(vp(nxt()), 1, vp(q), vp(sc), vp(zp), cl(tk), hd),
                 lambda: lib.hq_int8_quant_dynamic(vp(nxt()), 1, vp(q), vp(sc), vp(zp), tk, hd, None))):
            print(f"int8 quant {name} {tk}x{hd} fp16: reference kernel {timeit(rf, 200):.1f} us, libhq {timeit(of, 200):.1f} us")


if __name__ == "__main__":
    main()
