"""Bit-exact parity of hq_dequant_nf4 with the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def _run(hq, packed, absmax, n, blocksize, table=0):
    import torch
    dev = torch.device("cuda:0")
    out = hq.dequant_4bit(torch.from_numpy(packed).to(dev), torch.from_numpy(absmax).to(dev), n, blocksize, table)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("table", [0, 1])
@pytest.mark.parametrize("n,blocksize", [(4096 * 4096, 64), (4096 * 1100 + 8 * 37 + 3, 64), ((1 << 22) + 8, 256), (1 << 20, 128), (1 << 16, 4096), (96, 32),
                                         (100000, 64), (99999, 64), (31, 2), (4096, 16), (2048, 24), (64, 64)])
def test_bit_exact(hq, oracle, n, blocksize, table):
    packed, absmax = oa.make_nf4_problem(n + blocksize + table, n, blocksize)
    got = _run(hq, packed, absmax, n, blocksize, table)
    want = oracle.dequant_4bit(packed, absmax, n, blocksize, table).view(np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("pipe", [0, 1, 2, 8])
@pytest.mark.parametrize("n,blocksize", [(1 << 20, 64), (4096 * 1100 + 8 * 37 + 3, 64), (8, 8), (1032, 128), (100000, 64)])
def test_both_launch_variants(hq, oracle, tunable, n, blocksize, pipe):
    """The one-shot grid (by default only beyond 2^28 elements) and the persistent variant with one, two and
    eight workgroups per compute unit, forced on sizes from one word up: same bits."""
    tunable("HQ_NF4_PIPE", pipe)
    packed, absmax = oa.make_nf4_problem(n + pipe, n, blocksize)
    got = _run(hq, packed, absmax, n, blocksize, 0)
    want = oracle.dequant_4bit(packed, absmax, n, blocksize, 0).view(np.uint16)
    assert np.array_equal(got, want)


def test_all_codes_all_roundings(hq, oracle):
    """Every byte value against absmax values that exercise fp16 rounding,
    fp16 subnormal results and overflow to infinity."""
    absvals = np.array([1.0, 0.5, 2.0, 1.0009765625, 3.14159, 1e-4, 6.1e-5, 1e-7, 65504.0, 70000.0, 1e-30, 0.0],
                       np.float32)
    packed = np.tile(np.arange(256, dtype=np.uint8), absvals.size * 2)  # 512 elements per absmax
    n = packed.size * 2
    absmax = np.repeat(absvals, 2)  # blocksize 512: two blocks (all 256 byte values each) per value
    assert absmax.size * 512 == n
    for table in (0, 1):
        got = _run(hq, packed, absmax, n, 512, table)
        want = oracle.dequant_4bit(packed, absmax, n, 512, table).view(np.uint16)
        assert np.array_equal(got, want)


def test_nibble_order_and_special_codes(hq, oracle):
    """Byte 0xF0 -> [+absmax, -absmax]; code 7 -> +0 (NF4)."""
    packed = np.array([0xF0, 0x07, 0x70, 0x0F] * 8, np.uint8)
    absmax = np.array([1.5], np.float32)
    got = _run(hq, packed, absmax, 64, 64, 0).view(np.float16)
    assert got[0] == np.float16(1.5) and got[1] == np.float16(-1.5)
    assert got[2] == np.float16(-1.5) and got[3] == 0 and not np.signbit(got[3])
    assert got[4] == 0 and got[5] == np.float16(-1.5)
    assert got[6] == np.float16(-1.5) and got[7] == np.float16(1.5)


def test_empty(hq):
    import torch
    dev = torch.device("cuda:0")
    out = hq.dequant_4bit(torch.zeros(0, dtype=torch.uint8, device=dev), torch.zeros(0, device=dev), 0, 64)
    assert out.numel() == 0
