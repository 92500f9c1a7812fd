"""Bit-exact parity of the mxfp4 quantise-dequantise kernel with the CPU oracle and, where it was
built, with the reference kernel itself, through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def _tensor(bits, bf16):
    import torch
    t = torch.from_numpy(bits.view(np.int16).copy()).to("cuda:0")
    return t.view(torch.bfloat16 if bf16 else torch.float16)


def _bits(t):
    import torch
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def _random_bits(seed, n, bf16):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * np.exp2(rng.integers(-8, 8, n))).astype(np.float32)
    x[::53] = 0.0
    x[1::211] *= -0.0
    if bf16:
        return (x.view(np.uint32) >> 16).astype(np.uint16)
    return x.astype(np.float16).view(np.uint16)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("n", [32, 64, 4096, 32 * 1001, 1 << 20])
def test_bit_exact_vs_oracle(hq, oracle, n, bf16):
    import torch
    bits = _random_bits(n + bf16, n, bf16)
    got = hq.mxfp4_qdq(_tensor(bits, bf16))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(got), oracle.mxfp4_qdq(bits, bf16))


@pytest.mark.parametrize("bf16", [False, True])
def test_every_magnitude_below_saturation(hq, oracle, bf16):
    """Every bit pattern with magnitude up to 8 next to a 6 (scale 1) and next to a 4 (scale 1): the
    rounding function over its whole domain, both signs."""
    import torch
    pats = np.arange(65536, dtype=np.uint16)
    vals = (pats.astype(np.uint32) << 16).view(np.float32) if bf16 else pats.view(np.float16).astype(np.float32)
    keep = pats[np.isfinite(vals) & (np.abs(vals) <= 6.0)]
    for top in (6.0, 4.0):
        topbits = (np.array([top], np.float32).view(np.uint32) >> 16).astype(np.uint16) if bf16 else \
            np.array([top], np.float16).view(np.uint16)
        groups = np.full((len(keep), 32), 0, np.uint16)
        groups[:, 0] = topbits[0]
        groups[:, 1] = keep
        groups[:, 2:] = keep[:, None] ^ np.uint16(0x8000)      # the same magnitude with the other sign
        bits = groups.reshape(-1)
        got = hq.mxfp4_qdq(_tensor(bits, bf16))
        torch.cuda.synchronize()
        assert np.array_equal(_bits(got), oracle.mxfp4_qdq(bits, bf16))


@pytest.mark.parametrize("bf16", [False, True])
def test_group_maximum_rounding_past_the_format(hq, oracle, bf16):
    """Finite groups whose maximum rounds past the largest power of two of the format: the reference kernel
    writes NaN there (it takes log2 of an infinity); the library's documented behaviour is the finite scale
    2^14 (bf16: 2^126), the same as the oracle's."""
    import torch
    rng = np.random.default_rng(5)
    top = 0x7f7f if bf16 else 0x7bff
    lo = 0x7f60 if bf16 else 0x7b80
    bits = _random_bits(31, 32 * 64, bf16).reshape(-1, 32)
    bits[:, 0] = rng.integers(lo, top + 1, bits.shape[0]).astype(np.uint16)      # every group overflows the rounding
    bits[:, 1] = (bits[:, 0] - 0x0100) | 0x8000
    bits = bits.reshape(-1)
    got = _bits(hq.mxfp4_qdq(_tensor(bits, bf16)))
    torch.cuda.synchronize()
    want = oracle.mxfp4_qdq(bits, bf16)
    assert np.array_equal(got, want)
    inf = 0x7f80 if bf16 else 0x7c00
    assert ((got & 0x7fff) <= inf).all()          # no NaN anywhere


def test_empty_and_rejections(hq):
    import torch
    from hecbench_amd import HqError
    assert hq.mxfp4_qdq(torch.zeros(0, dtype=torch.float16, device="cuda:0")).numel() == 0
    with pytest.raises(HqError):
        hq.mxfp4_qdq(torch.zeros(48, dtype=torch.float16, device="cuda:0"))
    with pytest.raises(TypeError):
        hq.mxfp4_qdq(torch.zeros(64, dtype=torch.float32, device="cuda:0"))


@pytest.mark.parametrize("bf16", [False, True])
def test_vs_reference_kernel(hq, bf16):
    """The reference kernel on the same device buffer: bit-identical outputs on random data and on
    the reference main's own value set (src/mxfp4-hip/main.cu:181-195)."""
    import torch
    ref = oa.load_ref_hip()
    if ref is None or not hasattr(ref, "ref_mxfp4_qdq"):
        pytest.skip("oracle/_ref was not built with the mxfp4 kernel")
    n = 1 << 16
    rng = np.random.default_rng(123)
    v = np.array([0.0, 0.5, 1.0, 1.5, 2, 3, 4, -0.0, -0.5, -1.0, -1.5, -2, -3, -4, 0.25, 0.75, 1.25, 1.75, 2.5,
                  3.5, 5, 0.1, 0.3, 0.4, 0.6, 0.9, -0.1, -0.3, -0.4, -0.6, -0.9], np.float32)
    fixture = v[rng.integers(0, len(v), n)].reshape(-1, 32)
    pos = rng.integers(0, 32, fixture.shape[0])
    fixture[np.arange(fixture.shape[0]), pos] = np.where(pos < 16, 6.0, -6.0)
    fixture = fixture.reshape(-1)
    fbits = (fixture.view(np.uint32) >> 16).astype(np.uint16) if bf16 else fixture.astype(np.float16).view(np.uint16)
    for bits in (fbits, _random_bits(9, n, bf16)):
        # groups whose maximum rounds to zero are where the two differ by design (zero scale)
        grp = bits.reshape(-1, 32) & 0x7fff
        bits = bits.reshape(-1, 32)[grp.max(axis=1) >= (0x0400 if not bf16 else 0x0080)].reshape(-1)
        bits = bits[: (bits.size // 64) * 64]
        x = _tensor(bits, bf16)
        got = hq.mxfp4_qdq(x)
        theirs = torch.empty_like(x)
        ref.ref_mxfp4_qdq(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(theirs.data_ptr()), ctypes.c_int(bits.size),
                          ctypes.c_int(int(bf16)), None)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(got), _bits(theirs))
