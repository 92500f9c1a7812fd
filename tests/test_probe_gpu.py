"""The memory-system probes of the benchmark report: the copy mode copies, the read mode and the gather probe leave
their sinks alone, the gather count matches the launch, bad arguments are rejected before any launch."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


def _vp(t):
    return ctypes.c_void_p(t.data_ptr())


def test_stream_probe_copies_and_reads(hq):
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for n in (16, 4096, 1 << 20, (1 << 22) + 48):
        src = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda:0")
        dst = torch.zeros(n, dtype=torch.uint8, device="cuda:0")
        assert lib.hq_probe_stream(1, _vp(src), _vp(dst), n, st) == 0
        torch.cuda.synchronize()
        assert torch.equal(src, dst), n
        dst.fill_(7)
        assert lib.hq_probe_stream(0, _vp(src), _vp(dst), n, st) == 0     # read only: dst untouched
        torch.cuda.synchronize()
        assert bool((dst == 7).all()), n
    assert lib.hq_probe_stream(2, _vp(src), _vp(dst), 16, st) < 0        # unknown mode
    assert lib.hq_probe_stream(0, _vp(src), _vp(dst), 24, st) < 0        # not a multiple of 16
    assert lib.hq_probe_stream(0, None, _vp(dst), 16, st) < 0
    assert lib.hq_probe_stream(1, ctypes.c_void_p(src.data_ptr() + 4), _vp(dst), 16, st) < 0   # misaligned


def test_gather_probe(hq):
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    table = torch.randint(0, 256, (1 << 20,), dtype=torch.uint8, device="cuda:0")
    sink = torch.full((16,), 9, dtype=torch.uint8, device="cuda:0")
    want = 1 << 20
    cnt = lib.hq_probe_gather16_count(want)
    cus = hq.device_info()["compute_units"]
    assert cnt >= want and cnt % (cus * 8 * 256 * 8) == 0
    assert lib.hq_probe_gather16(_vp(table), 1 << 20, want, _vp(sink), st) == 0
    torch.cuda.synchronize()
    assert bool((sink == 9).all())
    assert lib.hq_probe_gather16(_vp(table), (1 << 20) - 16, want, _vp(sink), st) < 0   # not a power of two
    assert lib.hq_probe_gather16(_vp(table), 1 << 20, 0, _vp(sink), st) < 0
    assert lib.hq_probe_gather16(None, 1 << 20, want, _vp(sink), st) < 0


def test_lds_probe(hq):
    """Every pattern the benchmark runs is valid for the probe and leaves the sink alone; a conflict-free
    pattern is faster than the one that puts a whole pass into one bank; bad arguments are rejected."""
    import torch
    import bench
    from hecbench_amd import _lib
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.full((16,), 5, dtype=torch.uint8, device="cuda:0")
    for name, width, write, offs in bench.lds_patterns():
        table = torch.tensor(offs, dtype=torch.int32, device="cuda:0")
        assert lib.hq_probe_lds(_vp(table), width, write, 64, _vp(sink), st) == 0, name
    torch.cuda.synchronize()
    assert bool((sink == 5).all())
    res = {p["name"]: p["us_per_launch"] for p in bench.lds_probe(repeats=2048, launches=5)["patterns"]}
    assert res["read b32, 128 bytes apart (a pass in one bank)"] > 1.5 * res["read b32, consecutive words"], res
    table = torch.zeros(64, dtype=torch.int32, device="cuda:0")
    assert lib.hq_probe_lds(_vp(table), 48, 0, 64, _vp(sink), st) < 0        # no such width
    assert lib.hq_probe_lds(_vp(table), 32, 0, 0, _vp(sink), st) < 0         # no repeats
    assert lib.hq_probe_lds(None, 32, 0, 64, _vp(sink), st) < 0
    assert lib.hq_probe_lds(_vp(table), 32, 0, 64, None, st) < 0
