"""numpy-facing binding of the CPU oracle (oracle/libhq_oracle.so) and, where it
was built, of the reference compiled from its own sources (oracle/_ref/).
Test infrastructure: the product package never imports this module."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_SO = os.path.join(ORACLE_DIR, "libhq_oracle.so")
REF_CPU_SO = os.path.join(ORACLE_DIR, "_ref", "libhecref_cpu.so")
REF_HIP_SO = os.path.join(ORACLE_DIR, "_ref", "libhecref_hip.so")

_vp = ctypes.c_void_p


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


class Oracle:
    def __init__(self, lib):
        self.lib = lib
        lib.hqo_f32_to_f16.restype = ctypes.c_uint16
        lib.hqo_f32_to_f16.argtypes = [ctypes.c_float]
        lib.hqo_f16_to_f32.restype = ctypes.c_float
        lib.hqo_f16_to_f32.argtypes = [ctypes.c_uint16]
        lib.hqo_hfma.restype = ctypes.c_uint16
        lib.hqo_hfma.argtypes = [ctypes.c_uint16] * 3
        lib.hqo_dquantize.restype = ctypes.c_uint8
        lib.hqo_dquantize.argtypes = [_vp, ctypes.c_float]
        self.nf4_table = np.ctypeslib.as_array((ctypes.c_float * 16).in_dll(lib, "hqo_nf4_table")).copy()
        self.fp4_table = np.ctypeslib.as_array((ctypes.c_float * 16).in_dll(lib, "hqo_fp4_table")).copy()

    def set_threads(self, n):
        """Threads for the loops over independent outputs (1 = serial); results do not depend on it."""
        self.lib.hqo_set_threads(int(n))

    def max_threads(self):
        return int(self.lib.hqo_max_threads())

    # ---- q3
    def q3_pack(self, codes):
        K, N = codes.shape
        codes = np.ascontiguousarray(codes, np.uint8)
        mat = np.zeros((3 * K // 32, N), np.int32)
        self.lib.hqo_q3_pack(_p(codes), K, N, _p(mat))
        return mat

    def q3_unpack(self, mat, K):
        N = mat.shape[1]
        mat = np.ascontiguousarray(mat, np.int32)
        codes = np.zeros((K, N), np.uint8)
        self.lib.hqo_q3_unpack(_p(mat), K, N, _p(codes))
        return codes

    def q3_matvec_f32(self, x, mat, scales, zeros, mul=None):
        K, N = x.size, mat.shape[1]
        mul = np.zeros(N, np.float32) if mul is None else mul
        self.lib.hqo_q3_matvec_f32(_p(np.ascontiguousarray(x, np.float32)), _p(mat), _p(mul), _p(scales),
                                   _p(zeros), K, N)
        return mul

    def q3_matvec_f32_omp(self, x, mat, scales, zeros, mul=None):
        """Returns (result, threads used)."""
        K, N = x.size, mat.shape[1]
        mul = np.zeros(N, np.float32) if mul is None else mul
        threads = self.lib.hqo_q3_matvec_f32_omp(_p(np.ascontiguousarray(x, np.float32)), _p(mat), _p(mul),
                                                 _p(scales), _p(zeros), K, N)
        return mul, threads

    def q3_matvec_f64(self, x, mat, scales, zeros):
        K, N = x.size, mat.shape[1]
        y = np.zeros(N, np.float64)
        xd = np.ascontiguousarray(x, np.float64)
        self.lib.hqo_q3_matvec_f64(_p(xd), _p(mat), _p(y), _p(scales), _p(zeros), K, N)
        return y

    def q3_matvec_f16(self, x16, mat, scales, zeros, mul=None):
        K, N = x16.size, mat.shape[1]
        mul = np.zeros(N, np.float32) if mul is None else mul
        xb = np.ascontiguousarray(x16, np.float16).view(np.uint16)
        self.lib.hqo_q3_matvec_f16(_p(xb), _p(mat), _p(mul), _p(scales), _p(zeros), K, N)
        return mul

    def q3_gemm(self, A16, mat, scales, zeros, mode=0):
        M, K = A16.shape
        N = mat.shape[1]
        out = np.zeros((M, N), np.float64)
        Ab = np.ascontiguousarray(A16, np.float16).view(np.uint16)
        self.lib.hqo_q3_gemm(_p(Ab), _p(mat), _p(out), _p(scales), _p(zeros), M, K, N, mode)
        return out

    # ---- 4-bit dequant
    def dequant_4bit(self, packed, absmax, n, blocksize, table=0):
        out = np.zeros(n, np.uint16)
        self.lib.hqo_dequant_4bit(_p(packed), _p(absmax), _p(out), ctypes.c_int64(n), blocksize, table)
        return out.view(np.float16)

    def quantize_4bit(self, x, blocksize, table=0):
        n = x.size
        is16 = x.dtype == np.float16
        xb = np.ascontiguousarray(x).view(np.uint16) if is16 else np.ascontiguousarray(x, np.float32)
        packed = np.zeros((n + 1) // 2, np.uint8)
        absmax = np.zeros((n + blocksize - 1) // blocksize, np.float32)
        self.lib.hqo_quantize_4bit(_p(xb), int(is16), _p(packed), _p(absmax), ctypes.c_int64(n), blocksize, table)
        return packed, absmax

    # ---- dynamic 8-bit
    def dynamic_map(self):
        code = np.zeros(256, np.float32)
        self.lib.hqo_dynamic_map(_p(code))
        return code

    def quantize_dynamic8(self, code, A):
        A = np.ascontiguousarray(A, np.float32)
        out = np.zeros(A.size, np.uint8)
        self.lib.hqo_quantize_dynamic8(_p(code), _p(A), _p(out), ctypes.c_int64(A.size))
        return out

    # ---- int8 activation quantisation
    @staticmethod
    def _act(x):
        import torch  # bf16 arrays arrive as torch tensors (numpy has no bfloat16)
        if isinstance(x, torch.Tensor):
            assert x.dtype == torch.bfloat16
            return np.ascontiguousarray(x.view(torch.int16).numpy()).view(np.uint16), 2
        if x.dtype == np.float16:
            return np.ascontiguousarray(x).view(np.uint16), 1
        return np.ascontiguousarray(x, np.float32), 0

    def int8_quant_static(self, x, scale, azp=None):
        xb, dt = self._act(x)
        out = np.zeros(x.shape, np.int8)
        self.lib.hqo_int8_quant_static(_p(xb), dt, _p(out), ctypes.c_int64(x.shape[0]), int(x.shape[1]),
                                       ctypes.c_float(scale), 0 if azp is None else 1, 0 if azp is None else int(azp))
        return out

    def int8_quant_dynamic(self, x, with_azp=False):
        xb, dt = self._act(x)
        out = np.zeros(x.shape, np.int8)
        scales = np.zeros(x.shape[0], np.float32)
        azp = np.zeros(x.shape[0], np.int32) if with_azp else None
        self.lib.hqo_int8_quant_dynamic(_p(xb), dt, _p(out), _p(scales), _p(azp), ctypes.c_int64(x.shape[0]),
                                        int(x.shape[1]))
        return out, scales, azp

    # ---- gemv
    def gemv(self, mat, mode, vec16, scale=1.0, zero_point=0.0):
        """mode 0 fp16 / 1 int8 / 2 packed int4; returns (fp16 result, double result)."""
        rows = mat.shape[0]
        n = vec16.size
        mat = np.ascontiguousarray(mat)
        r16 = np.zeros(rows, np.uint16)
        r64 = np.zeros(rows, np.float64)
        mp = mat.view(np.uint16) if mode == 0 else mat
        self.lib.hqo_gemv(_p(mp), mode, _p(vec16.view(np.uint16)), _p(r16), _p(r64), rows, n,
                          ctypes.c_float(scale), ctypes.c_float(zero_point))
        return r16.view(np.float16), r64

    # ---- mxfp4
    def mxfp4_qdq(self, bits, is_bf16):
        """bits: uint16 patterns of fp16 / bf16 values; returns the quantise-dequantised patterns."""
        bits = np.ascontiguousarray(bits, np.uint16)
        out = np.zeros_like(bits)
        self.lib.hqo_mxfp4_qdq(_p(bits), _p(out), ctypes.c_int64(bits.size), int(is_bf16))
        return out

    # ---- LUT-GEMM
    def bcq_pack(self, signs):
        K, nb, N = signs.shape
        signs = np.ascontiguousarray(signs, np.int8)
        bW = np.zeros((K // 32, nb, N), np.uint32)
        self.lib.hqo_bcq_pack(_p(signs), K, N, nb, _p(bW))
        return bW

    def bcq_dequant(self, bW, alpha16, qbias16, group):
        kw, nb, N = bW.shape
        K = kw * 32
        W = np.zeros((K, N), np.float64)
        self.lib.hqo_bcq_dequant(_p(bW), _p(alpha16.view(np.uint16)),
                                 _p(None if qbias16 is None else qbias16.view(np.uint16)), K, N, nb, group, _p(W))
        return W

    def lut_gemv_f64(self, bW, alpha16, qbias16, x16, group):
        kw, nb, N = bW.shape
        y = np.zeros(N, np.float64)
        self.lib.hqo_lut_gemv_f64(_p(bW), _p(alpha16.view(np.uint16)),
                                  _p(None if qbias16 is None else qbias16.view(np.uint16)),
                                  _p(x16.view(np.uint16)), _p(y), kw * 32, N, nb, group)
        return y

    def lut_gemv_f16(self, bW, alpha16, qbias16, x16, group):
        kw, nb, N = bW.shape
        y = np.zeros(N, np.uint16)
        self.lib.hqo_lut_gemv_f16(_p(bW), _p(alpha16.view(np.uint16)),
                                  _p(None if qbias16 is None else qbias16.view(np.uint16)),
                                  _p(x16.view(np.uint16)), _p(y), kw * 32, N, nb, group)
        return y.view(np.float16)

    # ---- AQLM
    def aqlm_matvec(self, codes, codebooks16, scales16, x16, sizes, stride_int4, mode=0):
        M = codes.shape[0]
        K = x16.size
        y16 = np.zeros(M, np.uint16)
        y64 = np.zeros(M, np.float64)
        sz = (ctypes.c_int * 4)(*sizes)
        self.lib.hqo_aqlm_matvec(_p(np.ascontiguousarray(codes, np.int16)), _p(codebooks16.view(np.uint16)),
                                 _p(None if scales16 is None else scales16.view(np.uint16)),
                                 _p(x16.view(np.uint16)), _p(y16), _p(y64), M, K, sz, stride_int4, mode)
        return y16.view(np.float16), y64


_oracle = None


def load_oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            subprocess.run(["make", "-C", ORACLE_DIR, "libhq_oracle.so"], check=True)
        _oracle = Oracle(ctypes.CDLL(ORACLE_SO))
    return _oracle


def load_ref_cpu():
    """The reference's host quantiser (None if oracle/_ref was not built)."""
    if not os.path.exists(REF_CPU_SO):
        return None
    lib = ctypes.CDLL(REF_CPU_SO)
    lib.ref_dquantize.restype = ctypes.c_uint8
    lib.ref_dquantize.argtypes = [ctypes.c_float]
    lib.ref_code_table.restype = ctypes.POINTER(ctypes.c_float)
    return lib


def load_ref_hip():
    """The reference's HIP kernels and host fixture loops (None if not built)."""
    if not os.path.exists(REF_HIP_SO):
        return None
    return ctypes.CDLL(REF_HIP_SO)


# ------------------------------------------------------------------ inputs

def make_q3_problem(seed, K, N, x_dtype=np.float32, batch=None):
    """Seeded GPTQ 3-bit problem in the shape of the benchmark's fixture: codes, scales, pre-multiplied zeros, activations."""
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 8, size=(K, N), dtype=np.uint8)
    scales = rng.uniform(0.005, 0.02, size=N).astype(np.float32)
    zeros = (scales * rng.integers(3, 5, size=N).astype(np.float32)).astype(np.float32)
    shape = (K,) if batch is None else (batch, K)
    x = rng.standard_normal(shape).astype(x_dtype)
    return codes, scales, zeros, x


def make_nf4_problem(seed, n, blocksize):
    rng = np.random.default_rng(seed)
    packed = rng.integers(0, 256, size=(n + 1) // 2, dtype=np.uint8)
    absmax = rng.uniform(0.5, 2.0, size=(n + blocksize - 1) // blocksize).astype(np.float32)
    return packed, absmax


def make_lut_problem(seed, K, N, nb, group, zero_bias=True):
    rng = np.random.default_rng(seed)
    bW = rng.integers(0, 2 ** 32, size=(K // 32, nb, N), dtype=np.uint64).astype(np.uint32)
    alpha = np.abs(rng.normal(0, 0.02, size=(K // group, nb, N))).astype(np.float16)
    if zero_bias:
        qbias = np.zeros((K // group, N), np.float16)
    else:
        qbias = rng.normal(0, 0.01, size=(K // group, N)).astype(np.float16)
    x = rng.standard_normal(K).astype(np.float16)
    return bW, alpha, qbias, x


def make_aqlm_problem(seed, M, K, ncb=1):
    rng = np.random.default_rng(seed)
    codes = rng.integers(-32768, 32768, size=(M, K // 8), dtype=np.int64).astype(np.int16)
    codebooks = rng.normal(0, 0.05, size=(ncb, 65536, 8)).astype(np.float16)
    scales = rng.uniform(0.5, 1.5, size=M).astype(np.float16)
    x = rng.standard_normal(K).astype(np.float16)
    return codes, codebooks, scales, x
