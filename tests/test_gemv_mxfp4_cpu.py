"""Pins of the gemv and mxfp4 oracles (no GPU): closed forms, the reference's own
verification table (src/mxfp4-cuda/verify.h), hand-derived scale cases and an independent
numpy restatement."""
import numpy as np
import pytest

from tests import oracle_api as oa


@pytest.fixture(scope="module")
def o():
    return oa.load_oracle()


# ------------------------------------------------------------------------------ gemv

def gemv_problem(seed, rows, n, mode):
    rng = np.random.default_rng(seed)
    vec = rng.uniform(0.0, 1.0, n).astype(np.float16)          # the reference fills U(0,1) (simple_tensor.h:80-84)
    if mode == 0:
        mat = rng.uniform(0.0, 1.0, (rows, n)).astype(np.float16)
    elif mode == 1:
        mat = rng.integers(-128, 128, (rows, n)).astype(np.int8)
    else:
        mat = rng.integers(0, 256, (rows, n // 2)).astype(np.uint8)
    return mat, vec


def dense_of(mat, mode):
    if mode == 2:   # low nibble first
        return np.stack([mat & 15, mat >> 4], axis=-1).reshape(mat.shape[0], -1).astype(np.float64)
    return mat.astype(np.float64)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_gemv_oracle_vs_numpy_fp64(o, mode):
    mat, vec = gemv_problem(5 + mode, 48, 512, mode)
    scale, zp = (1.0, 0.0) if mode == 0 else (0.0625, 0.01)
    r16, r64 = o.gemv(mat, mode, vec, scale, zp)
    sc = float(np.float16(scale)) if mode else 1.0
    z = float(np.float16(zp)) if mode else 0.0
    want = sc * ((dense_of(mat, mode) - z) @ vec.astype(np.float64))
    assert np.allclose(r64, want, rtol=1e-12, atol=1e-9)
    assert np.array_equal(r16.view(np.uint16), want.astype(np.float16).view(np.uint16))


def test_gemv_closed_forms(o):
    n = 256
    ones = np.ones(n, np.float16)
    # all-ones matrix times all-ones vector is n
    assert np.all(o.gemv(np.ones((4, n), np.float16), 0, ones)[1] == n)
    # int8: (q - zp) * scale summed n times; zero point rounded to fp16 first
    r = o.gemv(np.full((3, n), -7, np.int8), 1, ones, 0.5, 1.001)[1]
    assert np.allclose(r, 0.5 * n * (-7 - float(np.float16(1.001))), rtol=1e-13)
    # int4 nibble order: byte 0xF0 holds column 0 = 0 (low nibble) and column 1 = 15
    mat = np.zeros((1, n // 2), np.uint8)
    mat[0, 0] = 0xF0
    v = np.zeros(n, np.float16)
    v[0], v[1] = 2.0, 3.0
    assert o.gemv(mat, 2, v, 1.0, 0.0)[1][0] == 45.0
    v[0], v[1] = 3.0, 0.0
    assert o.gemv(mat, 2, v, 1.0, 0.0)[1][0] == 0.0


# ----------------------------------------------------------------------------- mxfp4

def as_bits(x, bf16):
    x = np.asarray(x, np.float32)
    if bf16:
        return (x.view(np.uint32) >> 16).astype(np.uint16)      # the test values are exact in bf16
    return x.astype(np.float16).view(np.uint16)


def from_bits(b, bf16):
    if bf16:
        return (b.astype(np.uint32) << 16).view(np.float32)
    return b.view(np.float16).astype(np.float32)


# src/mxfp4-cuda/verify.h: what the reference's own check demands of (input -> output) when the
# group holds a +-6, i.e. when the shared scale is 1
VERIFY_TABLE = {0.25: 0.0, 0.75: 1.0, 1.25: 1.0, 1.75: 2.0, 2.5: 2.0, 3.5: 4.0, 5.0: 4.0,
                0.0: 0.0, 0.5: 0.5, 1.0: 1.0, 1.5: 1.5, 2.0: 2.0, 3.0: 3.0, 4.0: 4.0, 6.0: 6.0,
                0.625: 0.5, 0.125: 0.0, 0.375: 0.5, 0.875: 1.0}


@pytest.mark.parametrize("bf16", [False, True])
def test_mxfp4_reference_verification_table(o, bf16):
    for sign in (1.0, -1.0):
        keys = sorted(VERIFY_TABLE)
        x = np.zeros(32, np.float32)
        x[:len(keys)] = sign * np.array(keys, np.float32)
        x[31] = 6.0 * sign
        got = from_bits(o.mxfp4_qdq(as_bits(x, bf16), bf16), bf16)
        want = np.zeros(32, np.float32)
        want[:len(keys)] = sign * np.array([VERIFY_TABLE[k] for k in keys], np.float32)
        want[31] = 6.0 * sign
        assert np.array_equal(got, want)
        assert np.array_equal(np.signbit(got), np.signbit(x))        # -0.1 -> -0, as verify.h asks


@pytest.mark.parametrize("bf16", [False, True])
def test_mxfp4_reference_fixture_values(o, bf16):
    """The value set of the reference main (src/mxfp4-hip/main.cu:181-195) with a +-6 per group:
    the inequalities of verify.h that are not exact table entries."""
    v = np.array([0.1, 0.3, 0.4, 0.6, 0.9, -0.1, -0.3, -0.4, -0.6, -0.9], np.float32)
    want = np.array([0.0, 0.5, 0.5, 0.5, 1.0, -0.0, -0.5, -0.5, -0.5, -1.0], np.float32)
    x = np.zeros(32, np.float32)
    x[:10] = v
    x[20] = -6.0
    if bf16:   # 0.1 etc. are not exact in bf16: truncate as the storage type would hold them
        x = from_bits(as_bits(x, True), True)
    got = from_bits(o.mxfp4_qdq(as_bits(x, bf16), bf16), bf16)
    assert np.array_equal(got[:10], want) and got[20] == -6.0


@pytest.mark.parametrize("bf16", [False, True])
def test_mxfp4_shared_scale_cases(o, bf16):
    """Hand-derived from the definition: max 7 = 1.75 * 4 carries to 2^3 (scale 2), max 3.4 stays at
    2^1 (scale 0.5), max 0.02 = 1.28 * 2^-6 gives scale 2^-8."""
    def run(vals):
        x = np.zeros(32, np.float32)
        x[:len(vals)] = vals
        return from_bits(o.mxfp4_qdq(as_bits(x, bf16), bf16), bf16)[:len(vals)]
    # scale 2: grid 0,1,2,3,4,6,8,12; 7 / 2 = 3.5 ties to 4 -> 8; 5 / 2 = 2.5 ties to 2 -> 4; 0.4 / 2 < 0.25 -> 0
    got = run([7.0, 5.0, 1.0, 0.4, -3.0])
    assert np.array_equal(got, np.array([8.0, 4.0, 1.0, 0.0, -3.0], np.float32))
    # 3.5 = 1.75 * 2 carries as well: scale 1, and 3.5 ties to 4
    assert np.array_equal(run([3.5, 1.25]), np.array([4.0, 1.0], np.float32))
    # scale 0.5: grid 0,.25,.5,.75,1,1.5,2,3; 3.375 / 0.5 = 6.75 saturates at 6 -> 3;
    # 1.25 / 0.5 = 2.5 ties to 2 -> 1; 0.125 / 0.5 = 0.25 ties to 0; 0.625 / 0.5 = 1.25 ties to 1 -> 0.5
    got = run([3.375, 1.25, 0.125, -0.625, 0.875])
    assert np.array_equal(got, np.array([3.0, 1.0, 0.0, -0.5, 1.0], np.float32))
    # max exactly a power of two 2^e: scale 2^(e-2), the maximum maps to 4 and is kept
    got = run([0.015625, 0.0078125, 0.001953125])     # 2^-6, 2^-7, 2^-9: scale 2^-8 -> 4, 2, 0.5
    assert np.array_equal(got, np.array([0.015625, 0.0078125, 0.001953125], np.float32))


def numpy_mxfp4(x32, bf16):
    """Independent restatement on float64: group max -> power of two with carry at 1.75 -> scale ->
    nearest grid point (ties to even index within the binade structure)."""
    x = x32.astype(np.float64).reshape(-1, 32)
    out = np.zeros_like(x)
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6])
    for g in range(x.shape[0]):
        m = np.abs(x[g]).max()
        if m == 0:
            out[g] = x[g] * 0
            continue
        e = int(np.floor(np.log2(m)))
        if m / 2.0 ** e >= 1.75:
            e += 1
        scale = 2.0 ** (e - 2)
        q = np.abs(x[g]) / scale
        idx = np.abs(q[:, None] - grid[None, :])
        res = np.empty(32)
        for i in range(32):
            d = idx[i]
            best = np.flatnonzero(d == d.min())
            if len(best) == 2:      # tie: the grid point with the even mantissa bit, i.e. even index
                best = [b for b in best if b % 2 == 0]
            res[i] = grid[best[0]]
        out[g] = np.copysign(res * scale, x[g])
    return out.reshape(-1).astype(np.float32)


@pytest.mark.parametrize("bf16", [False, True])
def test_mxfp4_vs_numpy_restatement(o, bf16):
    rng = np.random.default_rng(77 + bf16)
    x = (rng.standard_normal(32 * 400) * np.exp2(rng.integers(-6, 7, 32 * 400))).astype(np.float32)
    x[::97] = 0.0
    x = from_bits(as_bits(x, bf16) if not bf16 else (x.view(np.uint32) >> 16).astype(np.uint16), bf16)
    got = from_bits(o.mxfp4_qdq(as_bits(x, bf16), bf16), bf16)
    want = numpy_mxfp4(x, bf16)
    assert np.array_equal(got, want)
    # idempotent: quantising a quantised tensor changes nothing
    again = from_bits(o.mxfp4_qdq(as_bits(got, bf16), bf16), bf16)
    assert np.array_equal(again, got)


@pytest.mark.parametrize("bf16", [False, True])
def test_mxfp4_group_maximum_rounding_past_the_format(o, bf16):
    """A finite group maximum whose power-of-two rounding leaves the format (fp16 >= 61440, bf16 >= 0x7f60):
    the reference kernel rounds it to infinity, takes log2(inf) and writes NaN for the whole group
    (src/mxfp4-hip/main.cu:126-141).  This library documents a different, finite behaviour there: the scale
    is the power of two the carry would have produced, 2^14 (bf16: 2^126), and elements quantise against it
    as anywhere else (the maximum itself lands on 4 * scale, which overflows to infinity)."""
    top = 0x7f7f if bf16 else 0x7bff                       # largest finite value
    bits = np.zeros(64, np.uint16)
    bits[0] = top
    bits[1] = 0x7f00 if bf16 else 0x7800                   # 2^127 | 32768: scale * 2 -> kept
    bits[2] = (0x7e80 if bf16 else 0x7400) | 0x8000        # -2^126 | -16384: -scale -> kept
    bits[3] = 0x7e00 if bf16 else 0x7000                   # scale / 2 -> kept (0.5 is on the grid)
    bits[4] = 0x3f80 if bf16 else 0x3c00                   # 1.0: far below scale / 4 -> 0
    bits[32] = 0x3f80 if bf16 else 0x3c00                  # second group, ordinary: 1.0 is kept
    got = o.mxfp4_qdq(bits, bf16)
    inf = 0x7f80 if bf16 else 0x7c00
    assert got[0] == inf
    assert got[1] == bits[1] and got[2] == bits[2] and got[3] == bits[3]
    assert got[4] == 0 and not got[5:32].any()
    assert got[32] == bits[32]
