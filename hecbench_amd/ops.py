"""Operator-level wrappers: same names, argument meaning and error behaviour as
the reference launch wrappers, over the C ABI.  No arithmetic happens here: a
wrapper checks dtype, element count, contiguity and device of every tensor
against the problem sizes (the C ABI sees raw pointers and cannot), then makes
one library call."""
import ctypes

import torch

from . import _lib

NF4 = 0
FP4 = 1
_F32, _F16 = 0, 1
_ACCUMULATE = 1


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _names(dtypes):
    return " or ".join(str(d).replace("torch.", "") for d in dtypes)


def _chk(t, name, dtypes, numel=None, optional=False):
    """dtype, element count and contiguity of one argument (ValueError names the argument)."""
    if t is None:
        if optional:
            return
        raise ValueError(f"{name} is required")
    if not isinstance(t, torch.Tensor):
        raise ValueError(f"{name} must be a torch tensor")
    if t.dtype not in dtypes:
        raise ValueError(f"{name} must be {_names(dtypes)}, got {str(t.dtype).replace('torch.', '')}")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name} must hold {numel} elements, got {t.numel()} (shape {tuple(t.shape)})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _dev(*ts):
    """All tensors on one GPU, which must be the current device (the library launches there)."""
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("hecbench_amd operators take device tensors only (no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise ValueError(f"tensors on different devices ({dev} and {t.device})")
    if dev is not None and dev.index != torch.cuda.current_device():
        raise ValueError(f"tensors live on {dev} but the current device is cuda:{torch.cuda.current_device()}")


_I32 = (torch.int32,)
_U32 = (torch.int32, torch.uint32) if hasattr(torch, "uint32") else (torch.int32,)
_FP32 = (torch.float32,)
_FP16 = (torch.float16,)


def init():
    _lib.check(_lib.load().hq_init(), "hq_init")


def device_info():
    lib = _lib.load()
    v = [ctypes.c_int() for _ in range(5)]
    name = ctypes.create_string_buffer(256)
    _lib.check(lib.hq_device_info(*[ctypes.byref(x) for x in v], name, 256), "hq_device_info")
    return {"compute_units": v[0].value, "wavefront_size": v[1].value, "lds_bytes_per_cu": v[2].value,
            "memory_clock_khz": v[3].value, "memory_bus_bits": v[4].value, "name": name.value.decode()}


def q3_matvec(x, qweight, scales, zeros, out=None, accumulate=False):
    """y[n] = sum_k x[k]*(scales[n]*q[k][n] - zeros[n]); x fp32 or fp16 [K]."""
    _chk(x, "x", (torch.float32, torch.float16))
    _chk(qweight, "qweight", _I32)
    if qweight.dim() != 2:
        raise ValueError("qweight must be [3*K/32][N]")
    K = x.numel()
    N = qweight.shape[1]
    if qweight.shape[0] * 32 != 3 * K:
        raise ValueError("qweight must have 3*K/32 packed rows")
    _chk(scales, "scales", _FP32, N)
    _chk(zeros, "zeros", _FP32, N)
    _chk(out, "out", _FP32, N, optional=True)
    _dev(x, qweight, scales, zeros, out)
    if out is None:
        out = torch.empty(N, dtype=torch.float32, device=x.device)
    dt = _F16 if x.dtype == torch.float16 else _F32
    rc = _lib.load().hq_q3_matvec(_ptr(x), dt, _ptr(qweight), _ptr(scales), _ptr(zeros), _ptr(out), K, N, 1,
                                  _ACCUMULATE if accumulate else 0, _stream())
    _lib.check(rc, "hq_q3_matvec")
    return out


def vecquant3matmul(vec, mat, mul, scales, zeros, height=None, width=None):
    """Reference signature (src/quant3MatMul-hip/kernels.h:171-190): mul += vec @ W."""
    # view(-1) never copies: a non-contiguous mul raises instead of losing the "mul +=" result in a temporary
    q3_matvec(vec.reshape(-1), mat, scales, zeros, out=_flat_inplace(mul, "mul"), accumulate=True)


def _flat_inplace(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_contiguous():
        raise ValueError(f"{name} must be a contiguous tensor (it is updated in place)")
    return t.view(-1)


def vecquant3matmul_faster(vec, mat, mul, scales, zeros, height=None, width=None):
    """Reference signature (src/quant3MatMul-hip/kernels.h:193-217): fp16 vec, mul += vec @ W."""
    if vec.dtype != torch.float16:
        raise ValueError("vecquant3matmul_faster takes an fp16 vector")
    q3_matvec(vec.reshape(-1), mat, scales, zeros, out=_flat_inplace(mul, "mul"), accumulate=True)


def q3_gemm(A, qweight, scales, zeros, out=None):
    """out[m][n] = sum_k A[m][k]*(scales[n]*q[k][n] - zeros[n]); A fp16 [M][K]."""
    _chk(A, "A", _FP16)
    _chk(qweight, "qweight", _I32)
    if A.dim() != 2 or qweight.dim() != 2:
        raise ValueError("A must be [M][K] and qweight [3*K/32][N]")
    M, K = A.shape
    N = qweight.shape[1]
    if qweight.shape[0] * 32 != 3 * K:
        raise ValueError("qweight must have 3*K/32 packed rows")
    _chk(scales, "scales", _FP32, N)
    _chk(zeros, "zeros", _FP32, N)
    _chk(out, "out", _FP32, M * N, optional=True)
    _dev(A, qweight, scales, zeros, out)
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=A.device)
    rc = _lib.load().hq_q3_matvec(_ptr(A), _F16, _ptr(qweight), _ptr(scales), _ptr(zeros), _ptr(out), K, N, M,
                                  0, _stream())
    _lib.check(rc, "hq_q3_matvec(batch)")
    return out


def dequant_4bit(packed, absmax, n_elems, blocksize, table=NF4, out=None):
    if n_elems < 0 or blocksize <= 0:
        raise ValueError("n_elems must be >= 0 and blocksize > 0")
    _chk(packed, "packed", (torch.uint8,), (n_elems + 1) // 2)
    _chk(absmax, "absmax", _FP32, (n_elems + blocksize - 1) // blocksize)
    _chk(out, "out", _FP16, n_elems, optional=True)
    _dev(packed, absmax, out)
    if out is None:
        out = torch.empty(n_elems, dtype=torch.float16, device=packed.device)
    rc = _lib.load().hq_dequant_nf4(_ptr(packed), _ptr(absmax), _ptr(out), n_elems, blocksize, table, _stream())
    _lib.check(rc, "hq_dequant_nf4")
    return out


def dynamic_map():
    """The signed dynamic 8-bit map of bitsandbytes (7 exponent bits), 256 sorted fp32 values in [-1, 1]: the
    table the reference ships as a literal (src/quantBnB-cuda/code.h).  Returns a CPU tensor."""
    import numpy as np
    f32 = np.float32
    vals = []
    for i in range(7):
        items = (1 << i) + 1
        step = (f32(1.0) - f32(0.1)) / f32(items - 1)
        b = [f32(0.1) + step * f32(j) if j < items // 2 else f32(1.0) - step * f32(items - 1 - j) for j in range(items)]
        sc = f32(10.0 ** (-6 + i))
        for j in range(items - 1):
            mean = (b[j] + b[j + 1]) / f32(2.0)
            vals += [sc * mean, -(sc * mean)]
    vals += [f32(0.0), f32(1.0)]
    return torch.from_numpy(np.sort(np.array(vals, dtype=f32)))


def quantize_dynamic8(code, A, out=None):
    _chk(code, "code", _FP32, 256)
    _chk(A, "A", _FP32)
    _chk(out, "out", (torch.uint8,), A.numel(), optional=True)
    _dev(code, A, out)
    if out is None:
        out = torch.empty(A.numel(), dtype=torch.uint8, device=A.device)
    rc = _lib.load().hq_quantize_dynamic8(_ptr(code), _ptr(A), _ptr(out), A.numel(), _stream())
    _lib.check(rc, "hq_quantize_dynamic8")
    return out


def lut_matmul(x, bW, alpha, q_bias, group_size, out=None):
    """matmul(output, input, nqW, m) of src/lut-gemm-hip/kernels.cu:27-31.
    bW uint32/int32 [K/32][nb][N], alpha fp16 [K/G][nb][N], q_bias fp16 [K/G][N] or None."""
    _chk(x, "x", _FP16)
    _chk(bW, "bW", _U32)
    if bW.dim() != 3:
        raise ValueError("bW must be [K/32][nbits][N]")
    K = x.numel()
    nb, N = bW.shape[1], bW.shape[2]
    if group_size <= 0 or K % group_size or bW.shape[0] * 32 != K:
        raise ValueError("bW must have K/32 packed rows and group_size must divide K")
    _chk(alpha, "alpha", _FP16, (K // group_size) * nb * N)
    _chk(q_bias, "q_bias", _FP16, (K // group_size) * N, optional=True)
    _chk(out, "out", _FP16, N, optional=True)
    _dev(x, bW, alpha, q_bias, out)
    if out is None:
        out = torch.empty(N, dtype=torch.float16, device=x.device)
    rc = _lib.load().hq_lut_gemv(_ptr(bW), _ptr(alpha), _ptr(q_bias), _ptr(x), _ptr(out), K, N, nb, group_size,
                                 _stream())
    _lib.check(rc, "hq_lut_gemv")
    return out


def code1x16_matvec(codes, x, codebooks, codebook_a_sizes, codebook_stride_int4, scales=None, out=None):
    """code1x16_matvec of src/quantAQLM-hip/main.cu:103-139 (plus the optional row scale)."""
    _chk(codes, "codes", (torch.int16,))
    _chk(x, "x", _FP16)
    if codes.dim() != 2:
        raise ValueError("codes must be [M][K/8]")
    M = codes.shape[0]
    K = x.numel()
    if codes.shape[1] * 8 != K:
        raise ValueError("codes must hold K/8 codes per row")
    sizes_list = list(codebook_a_sizes)
    if len(sizes_list) != 4:
        raise ValueError("codebook_a_sizes must hold four row bounds")
    # code book of the last row: the first j with M-1 < codebook_a_sizes[j]
    ncb = next((j for j in range(4) if M - 1 < sizes_list[j]), 3) + 1
    _chk(codebooks, "codebooks", _FP16)
    if codebooks.numel() < (ncb - 1) * codebook_stride_int4 * 8 + 65536 * 8:
        raise ValueError(f"codebooks too small for {ncb} code book(s) of 65536 x 8 halves at the given stride")
    _chk(scales, "scales", _FP16, M, optional=True)
    _chk(out, "out", _FP16, M, optional=True)
    _dev(codes, x, codebooks, scales, out)
    if out is None:
        out = torch.empty(M, dtype=torch.float16, device=x.device)
    sizes = (ctypes.c_int * 4)(*codebook_a_sizes)
    rc = _lib.load().hq_aqlm_matvec(_ptr(codes), _ptr(codebooks), _ptr(scales), _ptr(x), _ptr(out), M, K, sizes,
                                    codebook_stride_int4, _stream())
    _lib.check(rc, "hq_aqlm_matvec")
    return out


def q3_pack(codes):
    """codes uint8 [K][N] (0..7) -> qweight int32 [3K/32][N]."""
    _chk(codes, "codes", (torch.uint8,))
    if codes.dim() != 2 or codes.shape[0] % 32:
        raise ValueError("codes must be [K][N] with K a multiple of 32")
    _dev(codes)
    K, N = codes.shape
    out = torch.empty((3 * K // 32, N), dtype=torch.int32, device=codes.device)
    _lib.check(_lib.load().hq_q3_pack(_ptr(codes), _ptr(out), K, N, _stream()), "hq_q3_pack")
    return out


def bcq_pack(signs):
    """signs int8 [K][nb][N] (> 0 means +1) -> bW int32 [K/32][nb][N]."""
    _chk(signs, "signs", (torch.int8,))
    if signs.dim() != 3 or signs.shape[0] % 32:
        raise ValueError("signs must be [K][nbits][N] with K a multiple of 32")
    _dev(signs)
    K, nb, N = signs.shape
    out = torch.empty((K // 32, nb, N), dtype=torch.int32, device=signs.device)
    _lib.check(_lib.load().hq_bcq_pack(_ptr(signs), _ptr(out), K, N, nb, _stream()), "hq_bcq_pack")
    return out


def quantize_4bit(x, blocksize, table=NF4):
    """x fp32/fp16 [n] -> (packed uint8 [ceil(n/2)], absmax fp32 [ceil(n/blocksize)])."""
    _chk(x, "x", (torch.float32, torch.float16))
    if blocksize <= 0:
        raise ValueError("blocksize must be > 0")
    _dev(x)
    n = x.numel()
    packed = torch.empty((n + 1) // 2, dtype=torch.uint8, device=x.device)
    absmax = torch.empty((n + blocksize - 1) // blocksize, dtype=torch.float32, device=x.device)
    rc = _lib.load().hq_quantize_4bit(_ptr(x), _F16 if x.dtype == torch.float16 else _F32, _ptr(packed), _ptr(absmax),
                                      n, blocksize, table, _stream())
    _lib.check(rc, "hq_quantize_4bit")
    return packed, absmax


def _act_dtype(x):
    if x.dtype == torch.float32:
        return 0
    if x.dtype == torch.float16:
        return 1
    if x.dtype == torch.bfloat16:
        return 2
    raise ValueError("activations must be fp32, fp16 or bf16")


def static_scaled_int8_quant(x, scale, azp=None, out=None):
    """static_scaled_int8_quant of src/quantVLLM-hip/main.cu:133-148; x [tokens][hidden]."""
    _chk(x, "x", (torch.float32, torch.float16, torch.bfloat16))
    if x.dim() != 2:
        raise ValueError("x must be [tokens][hidden]")
    _chk(out, "out", (torch.int8,), x.numel(), optional=True)
    _dev(x, out)
    tokens, hidden = x.shape
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.int8, device=x.device)
    rc = _lib.load().hq_int8_quant_static(_ptr(x), _act_dtype(x), _ptr(out), tokens, hidden, float(scale),
                                          0 if azp is None else 1, 0 if azp is None else int(azp), _stream())
    _lib.check(rc, "hq_int8_quant_static")
    return out


def dynamic_scaled_int8_quant(x, with_azp=False, out=None):
    """dynamic_scaled_int8_quant of src/quantVLLM-hip/main.cu:150-168; returns (out, scales, azp or None)."""
    _chk(x, "x", (torch.float32, torch.float16, torch.bfloat16))
    if x.dim() != 2:
        raise ValueError("x must be [tokens][hidden]")
    _chk(out, "out", (torch.int8,), x.numel(), optional=True)
    _dev(x, out)
    tokens, hidden = x.shape
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.int8, device=x.device)
    scales = torch.empty(tokens, dtype=torch.float32, device=x.device)
    azp = torch.empty(tokens, dtype=torch.int32, device=x.device) if with_azp else None
    rc = _lib.load().hq_int8_quant_dynamic(_ptr(x), _act_dtype(x), _ptr(out), _ptr(scales), _ptr(azp), tokens, hidden,
                                           _stream())
    _lib.check(rc, "hq_int8_quant_dynamic")
    return out, scales, azp


def gemv_fp16(mat, vec, out=None):
    """solve_gemv_with_params of src/gemv-hip/gemv.cu:94-133: res = mat @ vec (fp16 in, fp32 sums, fp16 out)."""
    _chk(mat, "mat", _FP16)
    if mat.dim() != 2:
        raise ValueError("mat must be [rows][n]")
    rows, n = mat.shape
    _chk(vec, "vec", _FP16, n)
    _chk(out, "out", _FP16, rows, optional=True)
    _dev(mat, vec, out)
    if out is None:
        out = torch.empty(rows, dtype=torch.float16, device=mat.device)
    rc = _lib.load().hq_gemv_fp16(_ptr(mat), _ptr(vec), _ptr(out), rows, n, _stream())
    _lib.check(rc, "hq_gemv_fp16")
    return out


def gemv_int8(mat, vec, scale, zero_point, out=None):
    """solve_gemv_int8_quantized_with_params of src/gemv-hip/gemv.cu:52-92 (mat int8 [rows][n])."""
    _chk(mat, "mat", (torch.int8,))
    if mat.dim() != 2:
        raise ValueError("mat must be [rows][n]")
    rows, n = mat.shape
    _chk(vec, "vec", _FP16, n)
    _chk(out, "out", _FP16, rows, optional=True)
    _dev(mat, vec, out)
    if out is None:
        out = torch.empty(rows, dtype=torch.float16, device=mat.device)
    rc = _lib.load().hq_gemv_int8(_ptr(mat), _ptr(vec), _ptr(out), rows, n, float(scale), float(zero_point),
                                  _stream())
    _lib.check(rc, "hq_gemv_int8")
    return out


def gemv_int4(mat, vec, scale, zero_point, out=None):
    """solve_gemv_int4_quantized_with_params of src/gemv-hip/gemv.cu:10-50 (mat uint8 [rows][n/2], low nibble
    first)."""
    _chk(mat, "mat", (torch.uint8,))
    if mat.dim() != 2:
        raise ValueError("mat must be [rows][n/2]")
    rows, half_n = mat.shape
    _chk(vec, "vec", _FP16, 2 * half_n)
    _chk(out, "out", _FP16, rows, optional=True)
    _dev(mat, vec, out)
    if out is None:
        out = torch.empty(rows, dtype=torch.float16, device=mat.device)
    rc = _lib.load().hq_gemv_int4(_ptr(mat), _ptr(vec), _ptr(out), rows, 2 * half_n, float(scale),
                                  float(zero_point), _stream())
    _lib.check(rc, "hq_gemv_int4")
    return out


def mxfp4_qdq(x, out=None):
    """mxfp4<T>() of src/mxfp4-hip/main.cu:144-171: microscaling fp4 quantise-dequantise of an fp16 / bf16 tensor
    whose element count is a multiple of 32."""
    if isinstance(x, torch.Tensor) and x.dtype not in (torch.float16, torch.bfloat16):
        raise TypeError("mxfp4_qdq takes fp16 or bf16 tensors")
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(out, "out", (x.dtype,), x.numel(), optional=True)
    _dev(x, out)
    if out is None:
        out = torch.empty_like(x)
    rc = _lib.load().hq_mxfp4_qdq(_ptr(x), _ptr(out), x.numel(), 1 if x.dtype == torch.float16 else 2, _stream())
    _lib.check(rc, "hq_mxfp4_qdq")
    return out
