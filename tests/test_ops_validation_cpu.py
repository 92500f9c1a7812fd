"""The operator wrappers reject wrongly typed or sized tensors before any pointer reaches the C ABI.
Runs without a GPU: dtype / size checks come first, the device check last, so a fully consistent set of
CPU tensors ends at "device tensors only"."""
import pytest
import torch

import hecbench_amd as hq

K, N = 64, 8


def _q3():
    return dict(x=torch.zeros(K), w=torch.zeros((6, N), dtype=torch.int32), s=torch.zeros(N), z=torch.zeros(N))


def test_q3_matvec_checks():
    a = _q3()
    with pytest.raises(ValueError, match="device tensors only"):
        hq.q3_matvec(a["x"], a["w"], a["s"], a["z"])
    with pytest.raises(ValueError, match="qweight must be int32"):
        hq.q3_matvec(a["x"], a["w"].to(torch.int64), a["s"], a["z"])
    with pytest.raises(ValueError, match="scales must be float32"):
        hq.q3_matvec(a["x"], a["w"], a["s"].half(), a["z"])
    with pytest.raises(ValueError, match="zeros must hold 8 elements"):
        hq.q3_matvec(a["x"], a["w"], a["s"], torch.zeros(N - 1))
    with pytest.raises(ValueError, match="out must hold 8 elements"):
        hq.q3_matvec(a["x"], a["w"], a["s"], a["z"], out=torch.zeros(N + 4))
    with pytest.raises(ValueError, match="x must be float32 or float16"):
        hq.q3_matvec(a["x"].double(), a["w"], a["s"], a["z"])
    with pytest.raises(ValueError, match="packed rows"):
        hq.q3_matvec(a["x"], a["w"][:3], a["s"], a["z"])


def test_reference_wrappers_refuse_a_copy_of_mul():
    """vecquant3matmul accumulates into mul: a non-contiguous mul would be flattened into a temporary
    and the result lost, so it is an error."""
    a = _q3()
    mul = torch.zeros((N, 2))[:, 0]
    assert not mul.is_contiguous()
    with pytest.raises(ValueError, match="mul must be a contiguous tensor"):
        hq.vecquant3matmul(a["x"], a["w"], mul, a["s"], a["z"])
    with pytest.raises(ValueError, match="mul must be a contiguous tensor"):
        hq.vecquant3matmul_faster(a["x"].half(), a["w"], mul, a["s"], a["z"])


def test_q3_gemm_checks():
    a = _q3()
    A = torch.zeros((4, K), dtype=torch.float16)
    with pytest.raises(ValueError, match="device tensors only"):
        hq.q3_gemm(A, a["w"], a["s"], a["z"])
    with pytest.raises(ValueError, match="A must be float16"):
        hq.q3_gemm(A.float(), a["w"], a["s"], a["z"])
    with pytest.raises(ValueError, match="packed rows"):
        hq.q3_gemm(A, torch.zeros((3, N), dtype=torch.int32), a["s"], a["z"])
    with pytest.raises(ValueError, match="out must hold 32 elements"):
        hq.q3_gemm(A, a["w"], a["s"], a["z"], out=torch.zeros((4, N - 1)))


def test_dequant_and_quantize_checks():
    packed = torch.zeros(64, dtype=torch.uint8)
    absmax = torch.zeros(2)
    with pytest.raises(ValueError, match="device tensors only"):
        hq.dequant_4bit(packed, absmax, 128, 64)
    with pytest.raises(ValueError, match="packed must hold 64 elements"):
        hq.dequant_4bit(packed[:32], absmax, 128, 64)
    with pytest.raises(ValueError, match="absmax must hold 2 elements"):
        hq.dequant_4bit(packed, torch.zeros(1), 128, 64)
    with pytest.raises(ValueError, match="absmax must be float32"):
        hq.dequant_4bit(packed, absmax.half(), 128, 64)
    with pytest.raises(ValueError, match="out must be float16"):
        hq.dequant_4bit(packed, absmax, 128, 64, out=torch.zeros(128))
    with pytest.raises(ValueError, match="code must hold 256 elements"):
        hq.quantize_dynamic8(torch.zeros(255), torch.zeros(16))
    with pytest.raises(ValueError, match="out must be uint8"):
        hq.quantize_dynamic8(torch.zeros(256), torch.zeros(16), out=torch.zeros(16, dtype=torch.int8))


def test_lut_and_aqlm_checks():
    Kl, Nl, nb, G = 128, 64, 3, 64
    x = torch.zeros(Kl, dtype=torch.float16)
    bW = torch.zeros((Kl // 32, nb, Nl), dtype=torch.int32)
    alpha = torch.zeros((Kl // G, nb, Nl), dtype=torch.float16)
    qb = torch.zeros((Kl // G, Nl), dtype=torch.float16)
    with pytest.raises(ValueError, match="device tensors only"):
        hq.lut_matmul(x, bW, alpha, qb, G)
    with pytest.raises(ValueError, match="alpha must hold 384 elements"):
        hq.lut_matmul(x, bW, alpha[:1], qb, G)
    with pytest.raises(ValueError, match="q_bias must be float16"):
        hq.lut_matmul(x, bW, alpha, qb.float(), G)
    with pytest.raises(ValueError, match="group_size must divide K"):
        hq.lut_matmul(x, bW, alpha, qb, 48)
    codes = torch.zeros((16, 8), dtype=torch.int16)
    xa = torch.zeros(64, dtype=torch.float16)
    cb = torch.zeros((65536, 8), dtype=torch.float16)
    with pytest.raises(ValueError, match="device tensors only"):
        hq.code1x16_matvec(codes, xa, cb, (16, 0, 0, 0), 65536)
    with pytest.raises(ValueError, match="codebooks too small for 2 code book"):
        hq.code1x16_matvec(codes, xa, cb, (8, 16, 0, 0), 65536)
    with pytest.raises(ValueError, match="codes must be int16"):
        hq.code1x16_matvec(codes.int(), xa, cb, (16, 0, 0, 0), 65536)
    with pytest.raises(ValueError, match="scales must hold 16 elements"):
        hq.code1x16_matvec(codes, xa, cb, (16, 0, 0, 0), 65536, scales=torch.zeros(15, dtype=torch.float16))


def test_gemv_and_int8_checks():
    mat = torch.zeros((4, 32), dtype=torch.float16)
    with pytest.raises(ValueError, match="vec must hold 32 elements"):
        hq.gemv_fp16(mat, torch.zeros(16, dtype=torch.float16))
    with pytest.raises(ValueError, match="mat must be int8"):
        hq.gemv_int8(mat, torch.zeros(32, dtype=torch.float16), 1.0, 0.0)
    with pytest.raises(ValueError, match="vec must hold 64 elements"):
        hq.gemv_int4(torch.zeros((4, 32), dtype=torch.uint8), torch.zeros(32, dtype=torch.float16), 1.0, 0.0)
    with pytest.raises(ValueError, match="out must hold 128 elements"):
        hq.static_scaled_int8_quant(torch.zeros((4, 32)), 0.1, out=torch.zeros((4, 16), dtype=torch.int8))
    with pytest.raises(TypeError):
        hq.mxfp4_qdq(torch.zeros(64))
    with pytest.raises(ValueError, match="device tensors only"):
        hq.mxfp4_qdq(torch.zeros(64, dtype=torch.float16))
