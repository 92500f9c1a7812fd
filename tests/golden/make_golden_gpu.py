"""Writes the golden fixtures that need the reference's DEVICE code: run on a GPU box with
oracle/_ref built (`make -C oracle ref` where the HeCBench tree is mounted).  The fixtures are
data only: seeded inputs and the outputs the reference's own kernels produce for them.

    python tests/golden/make_golden_gpu.py [output directory]

  mxfp4_reference_kernel.npz   qdq_mxfp4_kernel (src/mxfp4-hip/main.cu:109-142), fp16 and bf16
  gemv_reference_kernels.npz   gemv_fp16 / gemv_quantized_int8 / gemv_quantized_int4
                               (src/gemv-hip/kernels.h:66-311), 256 x 256, blocks (16, 4)
  q3_reference_kernels.npz     VecQuant3MatMulKernel and ...Faster (src/quant3MatMul-hip/kernels.h:12-169)
  aqlm_reference_kernel.npz    Code1x16MatVec (src/quantAQLM-hip/main.cu:29-101)
  quantvllm_reference_kernels.npz  the four int8 quantisation kernels (src/quantVLLM-hip/main.cu:11-131)
  kquantize_reference_kernel.npz   kQuantize (src/quantBnB-hip/main.cu:90-130) with the table of code.h
"""
import ctypes
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from tests import oracle_api as oa  # noqa: E402
from tests.test_gemv_mxfp4_cpu import gemv_problem  # noqa: E402


def vp(t):
    return ctypes.c_void_p(t.data_ptr())


def main():
    out_dir = sys.argv[1] if len(sys.argv) > 1 else HERE
    ref = oa.load_ref_hip()
    assert ref is not None, "build oracle/_ref first: make -C oracle ref"
    o = oa.load_oracle()
    dev = "cuda:0"
    rng = np.random.default_rng(2024)

    # ---- mxfp4: random data over 14 binades plus the reference main's value set with a +-6 per group
    fix = {}
    for name, bf16 in (("f16", False), ("bf16", True)):
        n = 8192
        x = (rng.standard_normal(n) * np.exp2(rng.integers(-7, 7, n))).astype(np.float32)
        v = np.array([0.0, 0.5, 1.0, 1.5, 2, 3, 4, -0.0, -0.5, -1.0, -1.5, -2, -3, -4, 0.25, 0.75, 1.25, 1.75, 2.5,
                      3.5, 5, 0.1, 0.3, 0.4, 0.6, 0.9, -0.1, -0.3, -0.4, -0.6, -0.9], np.float32)
        y = v[rng.integers(0, len(v), 4096)].reshape(-1, 32)
        pos = rng.integers(0, 32, y.shape[0])
        y[np.arange(y.shape[0]), pos] = np.where(pos < 16, 6.0, -6.0)
        allx = np.concatenate([x, y.reshape(-1)])
        t = torch.from_numpy(allx).to(dev).to(torch.bfloat16 if bf16 else torch.float16)
        res = torch.empty_like(t)
        ref.ref_mxfp4_qdq(vp(t), vp(res), ctypes.c_int(t.numel()), ctypes.c_int(int(bf16)), None)
        torch.cuda.synchronize()
        fix[f"in_{name}"] = t.view(torch.int16).cpu().numpy().view(np.uint16)
        fix[f"out_{name}"] = res.view(torch.int16).cpu().numpy().view(np.uint16)
    np.savez_compressed(os.path.join(out_dir, "mxfp4_reference_kernel.npz"), **fix)

    # ---- gemv: the reference default size and launch shape
    fix = {}
    n, bx, by = 256, 16, 4
    for mode, name in ((0, "fp16"), (1, "int8"), (2, "int4")):
        mat, vec = gemv_problem(900 + mode, n, n, mode)
        dm, dv = torch.from_numpy(mat).to(dev), torch.from_numpy(vec).to(dev)
        res = torch.zeros(n, dtype=torch.float16, device=dev)
        args = [vp(dm), vp(dv), vp(res), ctypes.c_uint(n)]
        if mode == 0:
            ref.ref_gemv_fp16(*args, ctypes.c_uint(bx), ctypes.c_uint(by), None)
        else:
            fn = ref.ref_gemv_int8 if mode == 1 else ref.ref_gemv_int4
            fn(*args, ctypes.c_float(0.0625), ctypes.c_float(0.01), ctypes.c_uint(bx), ctypes.c_uint(by), None)
        torch.cuda.synchronize()
        fix[f"mat_{name}"], fix[f"vec_{name}"], fix[f"res_{name}"] = mat, vec, res.cpu().numpy()
    np.savez_compressed(os.path.join(out_dir, "gemv_reference_kernels.npz"), **fix)

    # ---- GPTQ 3-bit matvec: both reference kernels (K, N multiples of 256 as they require)
    K, N = 1024, 512
    codes, scales, zeros, x = oa.make_q3_problem(4242, K, N)
    mat = o.q3_pack(codes)
    dmat, ds, dz = (torch.from_numpy(t).to(dev) for t in (mat, scales, zeros))
    dx = torch.from_numpy(x).to(dev)
    y32 = torch.zeros(N, device=dev)
    y16 = torch.zeros(N, device=dev)
    ref.ref_vecquant3matmul_f32(vp(dx), vp(dmat), vp(y32), vp(ds), vp(dz), 3 * K // 32, N)
    ref.ref_vecquant3matmul_faster(vp(dx.half()), vp(dmat), vp(y16), vp(ds), vp(dz), 3 * K // 32, N)
    torch.cuda.synchronize()
    np.savez_compressed(os.path.join(out_dir, "q3_reference_kernels.npz"), mat=mat, scales=scales, zeros=zeros, x=x,
                        y_f32_kernel=y32.cpu().numpy(), y_faster_kernel=y16.cpu().numpy())

    # ---- AQLM: the reference kernel without scales, two code books.  Only 512 entries per code book are
    # used (256 at each end of the unsigned index range, so negative codes are covered); the fixture
    # stores those entries, the rest of the 65536 x 8 code books is zero.
    M, Kq = 256, 512
    used = np.concatenate([np.arange(0, 256), np.arange(65280, 65536)]).astype(np.int64)
    vals = rng.normal(0, 0.05, size=(2, used.size, 8)).astype(np.float16)
    cb = np.zeros((2, 65536, 8), np.float16)
    cb[:, used, :] = vals
    codes = used[rng.integers(0, used.size, size=(M, Kq // 8))].astype(np.uint16).view(np.int16)
    xa = rng.standard_normal(Kq).astype(np.float16)
    dc, dcb, dxa = (torch.from_numpy(t).to(dev) for t in (codes, cb, xa))
    ya = torch.zeros(M, dtype=torch.float16, device=dev)
    sizes = (ctypes.c_int * 4)(128, 256, 0, 0)
    ref.ref_code1x16_launch(vp(dc), vp(dxa), vp(ya), vp(dcb), M, Kq, sizes, 65536, None)
    torch.cuda.synchronize()
    np.savez_compressed(os.path.join(out_dir, "aqlm_reference_kernel.npz"), codes=codes, used_entries=used,
                        used_values=vals, x=xa, y=ya.cpu().numpy(), sizes=np.array([128, 256, 0, 0], np.int32))

    # ---- quantVLLM: the four device kernels on fp32 / fp16 / bf16 rows of 200 (fractions, the reference
    # main's integers, ties of x / 0.1), and kQuantize on normal draws plus every table entry and midpoint
    if hasattr(ref, "ref_hip_int8_quant_static"):
        from tests.test_oracle_cpu import _act_inputs
        fix = {}
        tokens, hidden = 24, 200
        for name, code in (("f32", 0), ("f16", 1), ("bf16", 2)):
            x = _act_inputs(name, tokens, hidden, 900 + code)
            dx = (x if isinstance(x, torch.Tensor) else torch.from_numpy(x)).to(dev)
            fix[f"x_{name}"] = (dx.view(torch.int16).cpu().numpy().view(np.uint16) if code == 2 else dx.cpu().numpy())
            for azp in (0, 54):
                q = torch.empty(tokens, hidden, dtype=torch.int8, device=dev)
                ref.ref_hip_int8_quant_static(vp(dx), code, vp(q), ctypes.c_long(tokens), hidden, ctypes.c_float(0.1), azp)
                torch.cuda.synchronize()
                fix[f"static_{name}_azp{azp}"] = q.cpu().numpy()
            for with_azp in (0, 1):
                q = torch.empty(tokens, hidden, dtype=torch.int8, device=dev)
                sc = torch.empty(tokens, device=dev)
                zp = torch.empty(tokens, dtype=torch.int32, device=dev)
                ref.ref_hip_int8_quant_dynamic(vp(dx), code, vp(q), vp(sc), vp(zp) if with_azp else None,
                                               ctypes.c_long(tokens), hidden)
                torch.cuda.synchronize()
                fix[f"dynamic_{name}_azp{with_azp}"] = q.cpu().numpy()
                fix[f"dynamic_{name}_azp{with_azp}_scales"] = sc.cpu().numpy()
                if with_azp:
                    fix[f"dynamic_{name}_azp1_zero_points"] = zp.cpu().numpy()
        np.savez_compressed(os.path.join(out_dir, "quantvllm_reference_kernels.npz"), **fix)
    ref.ref_hip_code_table.restype = ctypes.POINTER(ctypes.c_float)
    code = np.ctypeslib.as_array(ref.ref_hip_code_table(), shape=(256,)).copy()
    mids = ((code[:-1].astype(np.float64) + code[1:]) / 2).astype(np.float32)
    A = np.concatenate([rng.standard_normal(20000).astype(np.float32), code, mids,
                        np.nextafter(mids, np.float32(2)), np.nextafter(mids, np.float32(-2)),
                        np.array([-5, 5, 0, -0.0, 1e-30, -1e-30, np.inf, -np.inf], np.float32)])
    dA, dcode = torch.from_numpy(A).to(dev), torch.from_numpy(code).to(dev)
    qo = torch.zeros(A.size, dtype=torch.uint8, device=dev)
    ref.ref_kquantize(vp(dcode), vp(dA), vp(qo), ctypes.c_long(A.size), None)
    torch.cuda.synchronize()
    np.savez_compressed(os.path.join(out_dir, "kquantize_reference_kernel.npz"), code=code, A=A, out=qo.cpu().numpy())
    print("wrote fixtures to", out_dir)


if __name__ == "__main__":
    main()
