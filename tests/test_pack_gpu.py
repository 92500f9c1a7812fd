"""Device-side packers and the 4-bit quantiser against the CPU oracle (bit-exact), and
round trips through the matvec / dequant kernels, through the C ABI."""
import numpy as np
import pytest

from tests import oracle_api as oa
from tests.tol import rel_err

pytestmark = pytest.mark.gpu


def _t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


@pytest.mark.parametrize("K,N", [(4096, 1024), (32, 4), (96, 37), (1024, 11008)])
def test_q3_pack_bit_exact_and_round_trip(hq, oracle, K, N):
    import torch
    rng = np.random.default_rng(K + N)
    codes = rng.integers(0, 8, size=(K, N), dtype=np.uint8)
    got = hq.q3_pack(_t(codes))
    torch.cuda.synchronize()
    want = oracle.q3_pack(codes)
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.array_equal(oracle.q3_unpack(got.cpu().numpy(), K), codes)
    if N % 4 == 0:
        x = rng.integers(-8, 9, size=K).astype(np.float32)
        y = hq.q3_matvec(_t(x), got, _t(np.ones(N, np.float32)), _t(np.zeros(N, np.float32)))
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy().astype(np.int64), x.astype(np.int64) @ codes.astype(np.int64))


@pytest.mark.parametrize("K,N,nb", [(1024, 256, 3), (32, 5, 1), (256, 130, 8)])
def test_bcq_pack_bit_exact(hq, oracle, K, N, nb):
    import torch
    rng = np.random.default_rng(K + N + nb)
    signs = (rng.integers(0, 2, size=(K, nb, N)) * 2 - 1).astype(np.int8)
    got = hq.bcq_pack(_t(signs))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint32), oracle.bcq_pack(signs))


@pytest.mark.parametrize("table", [0, 1])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n,blocksize", [(4096 * 64, 64), (1000, 64), (999, 64), (4096, 128), (256, 2), (96, 32)])
def test_quantize_4bit_bit_exact_and_round_trip(hq, oracle, n, blocksize, dtype, table):
    import torch
    rng = np.random.default_rng(n + blocksize + table)
    x = (rng.standard_normal(n) * rng.uniform(0.01, 10)).astype(dtype)
    packed, absmax = hq.quantize_4bit(_t(x), blocksize, table)
    torch.cuda.synchronize()
    wp, wa = oracle.quantize_4bit(x, blocksize, table)
    assert np.array_equal(absmax.cpu().numpy(), wa)
    assert np.array_equal(packed.cpu().numpy(), wp)
    # round trip: dequantise on the GPU, compare with the oracle's dequantisation of the same codes
    deq = hq.dequant_4bit(packed, absmax, n, blocksize, table)
    torch.cuda.synchronize()
    want = oracle.dequant_4bit(wp, wa, n, blocksize, table)
    assert np.array_equal(deq.cpu().numpy().view(np.uint16), want.view(np.uint16))
    # and the round trip error is bounded by half the widest code gap times absmax
    err = np.abs(deq.cpu().numpy().astype(np.float32) - x.astype(np.float32))
    assert np.all(err <= 0.17 * np.repeat(wa, blocksize)[:n] + 1e-3 * np.abs(x.astype(np.float32)))


def test_zero_block_and_midpoint_ties(hq, oracle):
    import torch
    # an all-zero block has absmax 0 and code 7 (the zero entry); values exactly on a midpoint
    # take the lower code
    t = oracle.nf4_table
    mids = ((t[:-1] + t[1:]) * np.float32(0.5)).astype(np.float32)
    x = np.concatenate([np.zeros(64, np.float32), np.array([1.0], np.float32), mids, np.zeros(64 - 16, np.float32)])
    packed, absmax = hq.quantize_4bit(_t(x), 64, 0)
    torch.cuda.synchronize()
    wp, wa = oracle.quantize_4bit(x, 64, 0)
    assert np.array_equal(packed.cpu().numpy(), wp) and np.array_equal(absmax.cpu().numpy(), wa)
    codes = np.stack([wp >> 4, wp & 15], 1).reshape(-1)
    assert (codes[:64] == 7).all() and codes[64] == 15
    assert np.array_equal(codes[65:80], np.arange(15))
