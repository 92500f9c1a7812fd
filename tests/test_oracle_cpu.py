"""Pins of the CPU oracle: the reference's own known answers and host loops
(compiled from the reference tree into oracle/_ref where that tree is mounted),
closed forms, invariants and brute force.  Runs without a GPU."""
import ctypes
import os

import numpy as np
import pytest

from tests import oracle_api as oa


@pytest.fixture(scope="module")
def o():
    return oa.load_oracle()


# ------------------------------------------------------------------ fp16 helpers

def test_f16_conversion_matches_numpy_everywhere(o):
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16)
    back = np.array([o.lib.hqo_f16_to_f32(int(b)) for b in bits[::7]], np.float32)
    want = vals[::7].astype(np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(back[ok].view(np.uint32), want[ok].view(np.uint32)) and np.isnan(back[~ok]).all()
    rng = np.random.default_rng(0)
    f = np.concatenate([rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 4000),
                        np.array([0, -0.0, 65504, 65519.99, 65520, 1e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, np.inf],
                                 np.float32)])
    got = np.array([o.lib.hqo_f32_to_f16(float(v)) for v in f], np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(got, f.astype(np.float16).view(np.uint16))


def test_hfma_single_rounding(o):
    """a*b+c with one rounding: check against exact rational arithmetic."""
    from fractions import Fraction
    rng = np.random.default_rng(1)
    h = rng.standard_normal(3000).astype(np.float16).view(np.uint16)
    for a, b, c in zip(h[0::3], h[1::3], h[2::3]):
        exact = Fraction(float(np.uint16(a).view(np.float16))) * Fraction(float(np.uint16(b).view(np.float16))) \
            + Fraction(float(np.uint16(c).view(np.float16)))
        got = float(np.uint16(o.lib.hqo_hfma(int(a), int(b), int(c))).view(np.float16))
        # nearest fp16 to the exact value
        cand = np.float16(float(exact))
        lo, hi = np.nextafter(cand, np.float16(-np.inf)), np.nextafter(cand, np.float16(np.inf))
        best = min((abs(Fraction(float(v)) - exact), float(v)) for v in (lo, cand, hi))
        assert abs(Fraction(got) - exact) == best[0]


# ------------------------------------------------------------------ GPTQ 3-bit

def _reference_pattern(K, N):
    p1 = 0b01001001001001001001001001001001
    mat = np.zeros((3 * K // 32, N), np.uint32)
    mat[0::3] = p1
    mat[1::3] = (p1 << 1) & 0xFFFFFFFF
    mat[2::3] = (p1 << 2) & 0xFFFFFFFF
    return mat.view(np.int32)


def test_q3_reference_known_answer(o):
    """src/quant3MatMul-hip/main.cu:35-53,84-105: all codes 1, x=1, scale=-1, zero=0,
    K=49152 -> -49152 exactly, for the fp32 kernel and the fp16 'faster' kernel."""
    K, N = 49152, 64
    mat = _reference_pattern(K, N)
    assert (o.q3_unpack(mat, K) == 1).all()
    s, z = -np.ones(N, np.float32), np.zeros(N, np.float32)
    assert (o.q3_matvec_f32(np.ones(K, np.float32), mat, s, z) == -49152.0).all()
    assert (o.q3_matvec_f16(np.ones(K, np.float16), mat[:, :4].copy(), s[:4], z[:4]) == -49152.0).all()


def test_q3_pack_unpack_roundtrip_and_bit_positions(o):
    rng = np.random.default_rng(2)
    codes = rng.integers(0, 8, size=(128, 24), dtype=np.uint8)
    mat = o.q3_pack(codes)
    assert np.array_equal(o.q3_unpack(mat, 128), codes)
    # independent statement of the layout: 96-bit little-endian string, code i at bit 3i
    for n in (0, 7, 23):
        for g in range(4):
            big = sum(int(np.uint32(mat[3 * g + j, n])) << (32 * j) for j in range(3))
            assert [(big >> (3 * i)) & 7 for i in range(32)] == list(codes[32 * g:32 * g + 32, n])


def test_q3_matvec_closed_forms_and_dense(o):
    K, N = 512, 40
    rng = np.random.default_rng(3)
    # all codes = c, x = 1 -> y = K*(s*c - z)
    for c in (0, 3, 7):
        mat = o.q3_pack(np.full((K, N), c, np.uint8))
        s = rng.uniform(0.5, 2, N).astype(np.float32)
        z = rng.uniform(0.5, 2, N).astype(np.float32)
        want = K * (s.astype(np.float64) * c - z)
        assert np.allclose(o.q3_matvec_f64(np.ones(K), mat, s, z), want, rtol=1e-12)
    # dense double-precision matvec
    codes, s, z, x = oa.make_q3_problem(4, K, N)
    mat = o.q3_pack(codes)
    W = s[None, :].astype(np.float64) * codes - z[None, :]
    assert np.allclose(o.q3_matvec_f64(x, mat, s, z), x.astype(np.float64) @ W, rtol=1e-12, atol=1e-12)
    assert np.allclose(o.q3_matvec_f32(x, mat, s, z), x.astype(np.float64) @ W, rtol=1e-4, atol=1e-4)
    # exact integer case
    xi = rng.integers(-8, 9, K).astype(np.float32)
    y = o.q3_matvec_f32(xi, mat, np.ones(N, np.float32), np.zeros(N, np.float32))
    assert np.array_equal(y.astype(np.int64), xi.astype(np.int64) @ codes.astype(np.int64))
    # the OpenMP partition over columns changes nothing
    yo, threads = o.q3_matvec_f32_omp(x, mat, s, z)
    assert threads >= 1 and np.array_equal(yo, o.q3_matvec_f32(x, mat, s, z))
    # accumulate semantics of the reference (mul +=)
    y2 = o.q3_matvec_f32(xi, mat, np.ones(N, np.float32), np.zeros(N, np.float32), mul=np.full(N, 5, np.float32))
    assert np.array_equal(y2, y + 5)


def test_q3_f16_variant_close_to_exact(o):
    codes, s, z, x = oa.make_q3_problem(5, 512, 16, x_dtype=np.float16)
    mat = o.q3_pack(codes)
    y16 = o.q3_matvec_f16(x, mat, s, z)
    y64 = o.q3_matvec_f64(x.astype(np.float64), mat, s, z)
    assert np.max(np.abs(y16 - y64)) < 2e-2 * np.sqrt(np.mean(y64 ** 2))


def test_q3_gemm_rows_equal_matvec(o):
    codes, s, z, A = oa.make_q3_problem(6, 256, 32, x_dtype=np.float16, batch=5)
    mat = o.q3_pack(codes)
    out = o.q3_gemm(A, mat, s, z, mode=0)
    for m in range(5):
        assert np.allclose(out[m], o.q3_matvec_f64(A[m].astype(np.float64), mat, s, z), rtol=1e-12, atol=1e-12)
    out16 = o.q3_gemm(A, mat, s, z, mode=1)
    W16 = (s[None, :] * codes.astype(np.float32) - z[None, :]).astype(np.float16).astype(np.float64)
    assert np.allclose(out16, A.astype(np.float64) @ W16, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ NF4 / FP4

def test_nf4_table_is_the_qlora_construction(o):
    """NF4 = normalised quantiles of N(0,1) with offset 0.9677083 (QLoRA appendix)."""
    from scipy.stats import norm
    offset = 0.9677083
    pos = norm.ppf(np.linspace(offset, 0.5, 9)[:-1])
    neg = -norm.ppf(np.linspace(offset, 0.5, 8)[:-1])
    vals = np.sort(np.concatenate([pos, [0.0], neg]))
    vals /= np.abs(vals).max()
    assert np.allclose(o.nf4_table, vals, atol=2e-6)
    assert o.nf4_table[7] == 0 and o.nf4_table[0] == -1 and o.nf4_table[15] == 1
    assert (np.diff(o.nf4_table) > 0).all()


def test_dequant_4bit_properties(o):
    n, bs = 4096, 64
    packed, absmax = oa.make_nf4_problem(7, n, bs)
    out = o.dequant_4bit(packed, absmax, n, bs, 0)
    hi, lo = packed >> 4, packed & 15
    codes = np.stack([hi, lo], 1).reshape(-1)
    want = (o.nf4_table[codes] * np.repeat(absmax, bs)).astype(np.float32).astype(np.float16)
    assert np.array_equal(out.view(np.uint16), want.view(np.uint16))
    # nibble order: 0xF0 -> [+a, -a]
    out = o.dequant_4bit(np.array([0xF0], np.uint8), np.array([1.5], np.float32), 2, 64, 0)
    assert out[0] == np.float16(1.5) and out[1] == np.float16(-1.5)
    # FP4: sign bit 3, magnitudes {0, 1/192, 2/3, 1, 1/3, 1/2, 1/6, 1/4}
    mags = np.array([0, 1 / 192, 2 / 3, 1, 1 / 3, 1 / 2, 1 / 6, 1 / 4])
    assert np.allclose(np.abs(o.fp4_table[:8]), mags, rtol=1e-6)
    assert np.array_equal(o.fp4_table[8:], -o.fp4_table[:8])


def test_quantize_4bit_is_nearest_code_and_round_trips(o):
    rng = np.random.default_rng(12)
    n, bs = 4096, 64
    x = rng.standard_normal(n).astype(np.float32)
    for table, tab in ((0, o.nf4_table), (1, o.fp4_table)):
        packed, absmax = o.quantize_4bit(x, bs, table)
        assert np.array_equal(absmax, np.abs(x).reshape(-1, bs).max(1))
        codes = np.stack([packed >> 4, packed & 15], 1).reshape(-1)
        v = x / np.repeat(absmax, bs)
        d = np.abs(v[:, None].astype(np.float64) - tab[None, :].astype(np.float64))
        assert np.all(d[np.arange(n), codes] <= d.min(1) + 1e-6)   # brute-force nearest entry
        # dequantising the codes gives the nearest representable value, the block maximum exactly
        deq = o.dequant_4bit(packed, absmax, n, bs, table).astype(np.float32)
        assert np.max(np.abs(deq - x) / np.repeat(absmax, bs)) <= (0.17 if table == 0 else 0.17)
        big = np.abs(x) == np.repeat(absmax, bs)
        assert np.allclose(np.abs(deq[big]), absmax.astype(np.float16).astype(np.float32), rtol=0, atol=0)
    # idempotence: quantising the dequantised values reproduces the codes
    packed, absmax = o.quantize_4bit(x, bs, 0)
    deq32 = (o.nf4_table[np.stack([packed >> 4, packed & 15], 1).reshape(-1)] * np.repeat(absmax, bs)).astype(np.float32)
    p2, a2 = o.quantize_4bit(deq32, bs, 0)
    assert np.array_equal(p2, packed) and np.array_equal(a2, absmax)


# ------------------------------------------------------------------ dynamic 8-bit

def test_dquantize_against_reference_host_function(o):
    """The reference's own dQuantize<0> and code table (src/quantBnB-omp/main.cpp,
    src/quantBnB-cuda/code.h), compiled into oracle/_ref."""
    ref = oa.load_ref_cpu()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_cpu.so not built (reference tree not mounted)")
    code = np.ctypeslib.as_array(ref.ref_code_table(), shape=(256,)).copy()
    rng = np.random.default_rng(8)
    mids = ((code[:-1].astype(np.float64) + code[1:]) / 2).astype(np.float32)
    A = np.concatenate([rng.standard_normal(200000).astype(np.float32), code, mids,
                        np.nextafter(mids, np.float32(2)), np.nextafter(mids, np.float32(-2)),
                        np.array([-3, 3, 0, -0.0, 1, -1, 1e-30], np.float32)])
    want = np.zeros(A.size, np.uint8)
    ref.ref_dquantize_n(A.ctypes.data_as(ctypes.c_void_p), want.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(A.size))
    assert np.array_equal(o.quantize_dynamic8(code, A), want)


def test_dquantize_is_nearest_code(o):
    code = o.dynamic_map()
    assert code.size == 256 and (np.diff(code) > 0).all() and code[127] == 0 and code[255] == 1
    rng = np.random.default_rng(9)
    A = rng.uniform(-1, 1, 20000).astype(np.float32)
    got = o.quantize_dynamic8(code, A)
    d = np.abs(A[:, None].astype(np.float64) - code[None, :].astype(np.float64))
    best = d.min(1)
    # nearest entry up to the fp32 rounding of the midpoint test
    assert np.all(d[np.arange(A.size), got] <= best + 1e-7)
    assert np.array_equal(o.quantize_dynamic8(code, code), np.arange(256, dtype=np.uint8))


def test_dynamic_map_close_to_reference_table(o):
    ref = oa.load_ref_cpu()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_cpu.so not built (reference tree not mounted)")
    code = np.ctypeslib.as_array(ref.ref_code_table(), shape=(256,)).copy()
    # the generated map reproduces the reference table to 2 fp32 ulps (it is an INPUT of
    # the kernel, not part of its arithmetic: the bit-exact tests use the table they are given)
    assert np.all(np.abs(o.dynamic_map() - code) <= 2 * np.spacing(np.abs(code)))


def test_package_dynamic_map_equals_oracle(o):
    import hecbench_amd as hq
    assert np.array_equal(hq.dynamic_map().numpy(), o.dynamic_map())


# ------------------------------------------------------------------ LUT-GEMM

@pytest.mark.parametrize("fx,N,K,NB", [("ref_lut_fixture_256x256x3", 256, 256, 3),
                                       ("ref_lut_fixture_128x384x4", 128, 384, 4)])
def test_bcq_pack_and_dequant_against_reference_host_loops(o, fx, N, K, NB):
    """The reference's bit packing (main.cu:118-134) and host dequant loop
    dequantizeFrom_qW (main.cu:136-146), compiled into oracle/_ref."""
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built (reference tree not mounted)")
    G = K // 128
    qW = np.zeros((K, NB, N), np.float32)
    bW = np.zeros((K // 32, NB, N), np.uint32)
    alpha = np.zeros((G, NB, N), np.float32)
    qbias = np.zeros((G, N), np.float32)
    weight = np.zeros((N, K), np.float32)   # reference layout weight[n*K+k]
    inp = np.zeros(K, np.float32)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    getattr(ref, fx)(vp(qW), vp(bW), vp(alpha), vp(qbias), vp(weight), vp(inp))
    assert set(np.unique(qW)) == {-1.0, 1.0}
    assert np.array_equal(o.bcq_pack(qW.astype(np.int8)), bW)
    a16, b16 = alpha.astype(np.float16), qbias.astype(np.float16)
    W = o.bcq_dequant(bW, a16, b16, 128)
    # the reference loop works on the fp32 alphas; the oracle on their fp16 roundings
    want = np.zeros((K, N))
    for b in range(NB):
        want += np.repeat(a16.astype(np.float64)[:, b, :], 128, axis=0) * qW[:, b, :]
    want += np.repeat(b16.astype(np.float64), 128, axis=0)
    assert np.allclose(W, want, rtol=0, atol=1e-12)
    assert np.allclose(W, weight.T, atol=2e-3)  # fp32 alphas vs fp16 alphas
    x16 = inp.astype(np.float16)
    y = o.lut_gemv_f64(bW, a16, b16, x16, 128)
    assert np.allclose(y, x16.astype(np.float64) @ W, rtol=1e-12, atol=1e-12)


def test_lut_gemv_closed_forms(o):
    K, N, G = 256, 16, 128
    rng = np.random.default_rng(10)
    x = rng.integers(-4, 5, K).astype(np.float16)
    bW = rng.integers(0, 2 ** 32, size=(K // 32, 2, N), dtype=np.uint64).astype(np.uint32)
    qb = rng.integers(-2, 3, size=(K // G, N)).astype(np.float16)
    zero = np.zeros((K // G, 2, N), np.float16)
    y = o.lut_gemv_f64(bW, zero, qb, x, G)
    assert np.array_equal(y, (qb.astype(np.float64) * x.astype(np.float64).reshape(-1, G).sum(1)[:, None]).sum(0))
    # the reference's fp16 evaluation order agrees with the exact result on small integers
    one = np.ones((K // G, 2, N), np.float16)
    y16 = o.lut_gemv_f16(bW, one, qb, x, G)
    assert np.array_equal(y16.astype(np.float64), o.lut_gemv_f64(bW, one, qb, x, G))
    # LUT identity behind the kernel: entry(p) + entry(255 - p) = 0
    xs = x[:8].astype(np.float64)
    ent = lambda p: sum(xs[j] if (p >> j) & 1 else -xs[j] for j in range(8))
    assert all(ent(p) + ent(255 - p) == 0 for p in range(256))


# ------------------------------------------------------------------ AQLM

def test_aqlm_closed_forms(o):
    M, K = 12, 128
    rng = np.random.default_rng(11)
    x = rng.integers(-3, 4, K).astype(np.float16)
    codes = rng.integers(-32768, 32768, size=(M, K // 8), dtype=np.int64).astype(np.int16)
    ones = np.ones((1, 65536, 8), np.float16)
    y16, y64 = o.aqlm_matvec(codes, ones, None, x, (M, 0, 0, 0), 65536, mode=0)
    assert (y64 == x.astype(np.float64).sum()).all()
    y16b, _ = o.aqlm_matvec(codes, ones, None, x, (M, 0, 0, 0), 65536, mode=1)
    assert np.array_equal(y16, y16b)
    # signed storage, unsigned index: -1 -> 65535, -32768 -> 32768
    cb = np.zeros((1, 65536, 8), np.float16)
    cb[0, 65535, 0] = 1
    cb[0, 32768, 7] = 1
    c2 = np.zeros((2, K // 8), np.int16)
    c2[0], c2[1] = -1, -32768
    _, y = o.aqlm_matvec(c2, cb, None, x, (2, 0, 0, 0), 65536, mode=0)
    assert y[0] == x[0::8].astype(np.float64).sum() and y[1] == x[7::8].astype(np.float64).sum()
    # code book partition boundaries and brute force
    cb3 = rng.normal(0, 0.05, size=(3, 65536, 8)).astype(np.float16)
    sizes = (4, 8, 12, 100)
    sc = rng.uniform(0.5, 1.5, M).astype(np.float16)
    _, y = o.aqlm_matvec(codes, cb3, sc, x, sizes, 65536, mode=0)
    for m in range(M):
        book = cb3[m // 4].astype(np.float64)
        want = sum(book[int(np.uint16(codes[m, g]))] @ x[8 * g:8 * g + 8].astype(np.float64) for g in range(K // 8))
        assert np.isclose(y[m], want * float(sc[m]), rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ committed golden fixtures

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_golden_lut_fixture(o):
    """Bit planes, alphas, biases and dense weights written by the reference's own host
    loops (tests/golden/make_golden.py); needs neither the reference tree nor oracle/_ref."""
    f = np.load(os.path.join(GOLDEN, "lut_fixture_256x256x3.npz"))
    assert np.array_equal(o.bcq_pack(f["signs"]), f["bW"])
    a16, b16 = f["alpha"].astype(np.float16), f["q_bias"].astype(np.float16)
    W = o.bcq_dequant(f["bW"], a16, b16, 128)
    assert np.allclose(W, f["weight"].T, atol=2e-3)  # reference keeps fp32 alphas, the kernels fp16
    x16 = f["input"].astype(np.float16)
    y = o.lut_gemv_f64(f["bW"], a16, b16, x16, 128)
    assert np.allclose(y, x16.astype(np.float64) @ f["weight"].T.astype(np.float64), atol=5e-2)


def test_golden_dquantize_outputs(o):
    """Outputs of the reference host quantiser on a fixed vector.  The reference table is
    not committed; the generated dynamic map differs from it by at most 2 ulps in a few
    entries, which can move an input sitting within an ulp of a midpoint: allow 0.1%."""
    f = np.load(os.path.join(GOLDEN, "dquantize_outputs.npz"))
    got = o.quantize_dynamic8(o.dynamic_map(), f["A"])
    assert np.mean(got != f["out"]) <= 1e-3
    assert np.max(np.abs(got.astype(np.int32) - f["out"].astype(np.int32))) <= 1


# ------------------------------------------------------------------ int8 activation quantisation

def _act_inputs(dtype, tokens, hidden, seed):
    import torch
    rng = np.random.default_rng(seed)
    # the reference fixture (rand() % 1000 - 300) plus fractional values and a few extremes
    x = np.concatenate([rng.integers(-300, 700, size=(tokens // 2, hidden)).astype(np.float32),
                        (rng.standard_normal((tokens - tokens // 2, hidden)) * 37.3).astype(np.float32)])
    if hidden >= 4:
        x[0, :4] = [0.05, -0.05, 0.15, 12.75]  # ties of x / 0.1
    if dtype == "bf16":
        return torch.from_numpy(x).to(torch.bfloat16)
    return x.astype(np.float16 if dtype == "f16" else np.float32)


@pytest.mark.parametrize("dtype,code", [("f32", 0), ("f16", 1), ("bf16", 2)])
def test_int8_quant_against_reference_host_loops(o, dtype, code):
    """The four host loops of src/quantVLLM-cuda/reference.h, compiled into oracle/_ref."""
    ref = oa.load_ref_hip()
    if ref is None or not hasattr(ref, "ref_int8_quant_static"):
        pytest.skip("oracle/_ref/libhecref_hip.so not built (reference tree not mounted)")
    tokens, hidden = 24, 200
    x = _act_inputs(dtype, tokens, hidden, 3 + code)
    xb, _ = o._act(x)
    vp = lambda a: None if a is None else a.ctypes.data_as(ctypes.c_void_p)
    for azp in (None, 54, -200):
        want = np.zeros((tokens, hidden), np.int8)
        ref.ref_int8_quant_static(vp(xb), code, vp(want), ctypes.c_long(tokens), hidden, ctypes.c_float(0.1),
                                  0 if azp is None else 1, 0 if azp is None else azp)
        assert np.array_equal(o.int8_quant_static(x, 0.1, azp), want)
    for with_azp in (False, True):
        want = np.zeros((tokens, hidden), np.int8)
        ws = np.zeros(tokens, np.float32)
        wz = np.zeros(tokens, np.int32) if with_azp else None
        ref.ref_int8_quant_dynamic(vp(xb), code, vp(want), vp(ws), vp(wz), ctypes.c_long(tokens), hidden)
        got, gs, gz = o.int8_quant_dynamic(x, with_azp)
        assert np.array_equal(got, want) and np.array_equal(gs, ws)
        if with_azp:
            assert np.array_equal(gz, wz)


def test_int8_quant_closed_forms(o):
    x = np.array([[0.04, 0.05, 0.15, 0.25, -0.05, -0.15, 100.0, -100.0, 12.7, 12.75]], np.float32)
    q = o.int8_quant_static(x, 0.1)
    # 0.05/0.1 etc. are not exact in fp32; the saturating ends and clear cases are
    assert q[0, 0] == 0 and q[0, 6] == 127 and q[0, 7] == -128 and q[0, 8] == 127
    q, s, _ = o.int8_quant_dynamic(np.array([[1.0, -2.0, 0.5, 2.0]], np.float32))
    assert s[0] == np.float32(2.0) / np.float32(127.0) and list(q[0]) == [64, -127, 32, 127]
    q, s, z = o.int8_quant_dynamic(np.array([[0.0, 255.0, 127.5, 51.0]], np.float32), with_azp=True)
    assert s[0] == 1.0 and z[0] == -128 and list(q[0]) == [-128, 127, 0, -77]
