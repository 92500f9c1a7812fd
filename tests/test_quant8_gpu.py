"""Bit-exact parity of hq_quantize_dynamic8 with the CPU oracle, through the C ABI."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def _run(hq, code, A):
    import torch
    dev = torch.device("cuda:0")
    out = hq.quantize_dynamic8(torch.from_numpy(code).to(dev), torch.from_numpy(A).to(dev))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("n", [1 << 20, 1000003, 5, 256])
def test_bit_exact_normal_inputs(hq, oracle, n):
    code = oracle.dynamic_map()
    A = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    assert np.array_equal(_run(hq, code, A), oracle.quantize_dynamic8(code, A))


def test_table_values_midpoints_and_extremes(hq, oracle):
    code = oracle.dynamic_map()
    mids = ((code[:-1].astype(np.float64) + code[1:]) / 2).astype(np.float32)
    A = np.concatenate([code, mids, np.nextafter(mids, np.float32(2)), np.nextafter(mids, np.float32(-2)),
                        np.array([-5, 5, -1, 1, 0, -0.0, 1e-30, -1e-30, np.inf, -np.inf], np.float32)])
    assert np.array_equal(_run(hq, code, A), oracle.quantize_dynamic8(code, A))


def _probe_inputs(code, rng, extra=200000):
    """Inputs that sit on, between and just beside every table entry, at every scale down to the
    subnormals, beyond both ends, and the non-finite values, padded to a multiple of 4 with draws
    spread over the table's range."""
    c = code[np.isfinite(code)].astype(np.float32)
    mids = ((c[:-1].astype(np.float64) + c[1:]) / 2).astype(np.float32)
    pts = np.concatenate([c, mids])
    near = np.concatenate([pts, np.nextafter(pts, np.float32(np.inf)), np.nextafter(pts, np.float32(-np.inf))])
    scales = np.float32(2.0) ** np.arange(-150, 4, dtype=np.float32)
    span = float(np.max(np.abs(c))) if c.size else 1.0
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, -np.nan, 3.4e38, -3.4e38, 1e-45, -1e-45], np.float32)
    snan = np.array([0x7f800001, 0xff800001, 0x7fc00000, 0xffc12345], np.uint32).view(np.float32)
    draws = np.concatenate([rng.uniform(-1.2 * span, 1.2 * span, extra), rng.standard_normal(extra) * span,
                            rng.standard_normal(extra) * span * 1e-3, rng.standard_normal(extra) * span * 1e-6])
    with np.errstate(over="ignore"):
        A = np.concatenate([near, span * scales, -span * scales, special, snan, draws.astype(np.float32)])
    return np.ascontiguousarray(np.resize(A, (A.size + 3) // 4 * 4).astype(np.float32))


def _tables(oracle):
    rng = np.random.default_rng(5)
    dyn = oracle.dynamic_map()
    lin = np.linspace(-1, 1, 256, dtype=np.float32)
    dup = np.sort(rng.choice(np.linspace(-3, 3, 40, dtype=np.float32), 256))        # many equal neighbours
    tiny = np.sort(rng.standard_normal(256).astype(np.float32)) * np.float32(1e-20)
    big = np.sort(rng.standard_normal(256).astype(np.float32)) * np.float32(1e25)
    pos = np.sort(rng.uniform(0.5, 0.5001, 256).astype(np.float32))                 # one bucket holds every entry
    signed_zero = dyn.copy(); signed_zero[127] = -0.0
    zeros = np.zeros(256, np.float32)                                               # no magnitude: descent path
    shuffled = rng.permutation(dyn)                                                 # unsorted: descent path
    huge = np.sort(rng.standard_normal(256).astype(np.float32)) * np.float32(1e38)  # beyond the fast path's range
    with_inf = dyn.copy(); with_inf[0] = -np.inf; with_inf[255] = np.inf
    with_nan = dyn.copy(); with_nan[200] = np.nan
    logs = np.sort(np.concatenate([-np.logspace(-30, 0, 128), np.logspace(-30, 0, 128)]).astype(np.float32))
    return {"dynamic": dyn, "linear": lin, "duplicates": dup, "tiny": tiny, "big": big, "one_bucket": pos,
            "minus_zero_entry": signed_zero, "all_zero": zeros, "unsorted": shuffled, "huge": huge,
            "infinite_ends": with_inf, "nan_entry": with_nan, "log_spaced": logs}


@pytest.mark.parametrize("name", ["dynamic", "linear", "duplicates", "tiny", "big", "one_bucket", "minus_zero_entry",
                                  "all_zero", "unsorted", "huge", "infinite_ends", "nan_entry", "log_spaced"])
def test_bit_exact_over_tables(hq, oracle, name):
    """Sorted tables take the bucket-table path, the others the tree descent; both must give the
    reference's answer for every input, whatever the table's shape."""
    code = _tables(oracle)[name]
    A = _probe_inputs(code, np.random.default_rng(len(name)))
    got, want = _run(hq, code, A), oracle.quantize_dynamic8(code, A)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, (name, A[bad[:8]], got[bad[:8]], want[bad[:8]])


def test_vs_reference_kernel(hq, oracle):
    import torch
    ref = oa.load_ref_hip()
    if ref is None:
        pytest.skip("oracle/_ref/libhecref_hip.so not built")
    dev = torch.device("cuda:0")
    ref.ref_hip_code_table.restype = ctypes.POINTER(ctypes.c_float)
    code = np.ctypeslib.as_array(ref.ref_hip_code_table(), shape=(256,)).copy()
    n = 1 << 20
    A = np.random.default_rng(77).standard_normal(n).astype(np.float32)
    dA, dcode = torch.from_numpy(A).to(dev), torch.from_numpy(code).to(dev)
    out = torch.zeros(n, dtype=torch.uint8, device=dev)
    ref.ref_kquantize(ctypes.c_void_p(dcode.data_ptr()), ctypes.c_void_p(dA.data_ptr()),
                      ctypes.c_void_p(out.data_ptr()), ctypes.c_long(n), None)
    torch.cuda.synchronize()
    y = hq.quantize_dynamic8(dcode, dA)
    torch.cuda.synchronize()
    assert torch.equal(y, out)


def test_full_size_round_trip(hq):
    """At the benchmark's size, without the oracle: every table value quantises to its own index (the
    dynamic map is strictly increasing), and an input between two entries to one of the two."""
    import torch
    dev = torch.device("cuda:0")
    code = hq.dynamic_map().to(dev)
    n = 16777216
    g = torch.Generator(device=dev); g.manual_seed(5)
    idx = torch.randint(0, 256, (n,), device=dev, generator=g)
    out = hq.quantize_dynamic8(code, code[idx])
    assert torch.equal(out.long(), idx)
    x = torch.empty(n, device=dev).uniform_(-0.99, 0.99, generator=g)
    q = hq.quantize_dynamic8(code, x).long()
    lo = torch.searchsorted(code, x, right=True) - 1          # code[lo] <= x < code[lo + 1]
    assert bool(((q == lo) | (q == lo + 1)).all())
    nearest = torch.where((x - code[lo]).abs() <= (code[(lo + 1).clamp(max=255)] - x).abs(), lo, lo + 1)
    assert float((q != nearest).float().mean()) < 1e-4        # they differ on exact ties only
