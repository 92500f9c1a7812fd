"""Calls on different streams use different workspaces and may overlap: interleaved split-K
matvecs and batched GEMMs on two streams give the results of the same calls on one stream."""
import numpy as np
import pytest

from tests import oracle_api as oa

pytestmark = pytest.mark.gpu


def test_two_streams_interleaved(hq, oracle, tunable):
    import torch
    dev = torch.device("cuda:0")
    tunable("HQ_Q3_KSPLIT", 4)          # force the cross-workgroup reduction (workspace + counters)
    tunable("HQ_Q3_WAVES", 4)
    tunable("HQ_Q3_STEPS", 1)
    K, N, M = 2048, 512, 24
    problems = []
    for seed in (1, 2):
        codes, scales, zeros, x = oa.make_q3_problem(100 + seed, K, N)
        mat = oracle.q3_pack(codes)
        A = np.random.default_rng(seed).standard_normal((M, K)).astype(np.float16)
        problems.append(tuple(torch.from_numpy(t).to(dev) for t in (x, mat, scales, zeros, A)))
    # one stream, one call at a time
    want = []
    for x, mat, s, z, A in problems:
        want.append((hq.q3_matvec(x, mat, s, z).clone(), hq.q3_gemm(A, mat, s, z).clone()))
    torch.cuda.synchronize()
    # two streams, many interleaved calls in flight
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for rep in range(20):
        for i, st in enumerate(streams):
            x, mat, s, z, A = problems[i]
            with torch.cuda.stream(st):
                outs[i].append((hq.q3_matvec(x, mat, s, z), hq.q3_gemm(A, mat, s, z)))
    torch.cuda.synchronize()
    for i in range(2):
        for y, g in outs[i]:
            assert torch.equal(y, want[i][0])
            assert torch.equal(g, want[i][1])
