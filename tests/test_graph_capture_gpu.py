"""Calls recorded into a HIP graph: after hq_reserve_workspace the entry points that use a workspace (split-K
matvec, a small batch on the same split, batched GEMM) allocate nothing during capture, and hq_q3_matvec_noalloc never does.  Every replay is
checked against the eager result, with eager work and synchronisations between the replays."""
import ctypes

import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def _t(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def test_replays_match_eager(hq, oracle):
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    K, N = 8192, 8256                       # two rounds of K: split over two workgroups per tile (workspace)
    codes, scales, zeros, x = oa.make_q3_problem(901, K, N)
    mat = oracle.q3_pack(codes)
    Kg, Ng, M = 1024, 516, 72               # batched GEMM (more than 64 rows): pre-pass and main kernel meet in the workspace
    codes_g, scales_g, zeros_g, A = oa.make_q3_problem(902, Kg, Ng, x_dtype=np.float16, batch=M)
    mat_g = oracle.q3_pack(codes_g)
    dx, dm, ds, dz = _t(x), _t(mat), _t(scales), _t(zeros)
    dA, dmg, dsg, dzg = _t(A), _t(mat_g), _t(scales_g), _t(zeros_g)
    y = torch.zeros(N, device="cuda:0")
    y_na = torch.zeros(N, device="cuda:0")
    yg = torch.zeros(M, Ng, device="cuda:0")
    A4 = torch.randn(4, K, device="cuda:0").half()          # batch 4 on the matvec's weights: partial sums of four rows
    A24 = torch.randn(24, Kg, device="cuda:0").half()        # 24 rows on the small matrix: six row blocks per tile
    y24 = torch.zeros(24, Ng, device="cuda:0")
    y4 = torch.zeros(4, N, device="cuda:0")
    stream = torch.cuda.Stream()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())

    def noalloc(s):
        rc = lib.hq_q3_matvec_noalloc(vp(dx), 0, vp(dm), vp(ds), vp(dz), vp(y_na), K, N, 1, 0,
                                      ctypes.c_void_p(s.cuda_stream))
        assert rc == 0, rc

    with torch.cuda.stream(stream):
        assert lib.hq_reserve_workspace(ctypes.c_void_p(stream.cuda_stream), K, N) == 0
        hq.q3_matvec(dx, dm, ds, dz, out=y)
        hq.q3_gemm(dA, dmg, dsg, dzg, out=yg)
        hq.q3_gemm(A4, dm, ds, dz, out=y4)
        hq.q3_gemm(A24, dmg, dsg, dzg, out=y24)
        noalloc(stream)
    stream.synchronize()
    want, want_g, want_na, want_4, want_24 = y.clone(), yg.clone(), y_na.clone(), y4.clone(), y24.clone()
    assert torch.equal(want, want_na)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        hq.q3_matvec(dx, dm, ds, dz, out=y)
        hq.q3_gemm(dA, dmg, dsg, dzg, out=yg)
        hq.q3_gemm(A4, dm, ds, dz, out=y4)
        hq.q3_gemm(A24, dmg, dsg, dzg, out=y24)
        noalloc(torch.cuda.current_stream())
    for rep in range(4):
        y.fill_(float(rep)); yg.fill_(-1.0); y_na.fill_(7.0); y4.fill_(3.0); y24.fill_(5.0)  # eager work between the replays
        other = hq.q3_matvec(dx, dm, ds, dz)                       # an eager call on another stream's workspace
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), rep
        assert torch.equal(yg, want_g), rep
        assert torch.equal(y4, want_4), rep
        assert torch.equal(y24, want_24), rep
        assert torch.equal(y_na, want_na), rep
        assert torch.equal(other, want), rep


def test_capture_after_reserve_only(hq):
    """A fresh stream sees nothing but hq_reserve_workspace before the capture: every recorded call with a
    smaller K or N - among them a batched GEMM whose few column tiles split K, the largest workspace user -
    must find its workspace there (an allocation during capture would fail the call)."""
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    dev = "cuda:0"
    g = torch.Generator(device=dev)
    g.manual_seed(77)
    maxK, maxN = 8192, 8256
    shapes = [(1, 8192, 8256), (72, 8192, 4096), (4, 8192, 8256), (24, 1024, 516), (1, 4096, 1024), (16, 4096, 4096)]
    probs = []
    for M, K, N in shapes:
        mat = torch.randint(-2 ** 31, 2 ** 31 - 1, (3 * K // 32, N), dtype=torch.int32, device=dev, generator=g)
        s = torch.empty(N, device=dev).uniform_(0.005, 0.02, generator=g)
        z = s * torch.randint(3, 5, (N,), device=dev, generator=g).float()
        x = torch.randn(M, K, device=dev, generator=g)
        x = x[0].contiguous() if M == 1 else x.half()
        probs.append((M, x, mat, s, z))

    def run(p, out):
        M, x, mat, s, z = p
        return hq.q3_matvec(x, mat, s, z, out=out) if M == 1 else hq.q3_gemm(x, mat, s, z, out=out)

    # eager results on the default stream (this also sets the kernels' one-time function attributes)
    want = [run(p, None).clone() for p in probs]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    outs = [torch.zeros_like(w) for w in want]
    assert lib.hq_reserve_workspace(ctypes.c_void_p(stream.cuda_stream), maxK, maxN) == 0
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for p, o in zip(probs, outs):
            run(p, o)
    for rep in range(3):
        for o in outs:
            o.fill_(float(rep))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for (M, *_), o, w in zip(probs, outs, want):
            assert torch.equal(o, w), (rep, M, tuple(o.shape))
