"""Guard on the launch policy of hq_q3_matvec: on a handful of fixed shapes the plan the library picks by itself
must be within 10 % of the fastest candidate plan (each forced through hq_set_tunable and timed on rotated weight
buffers).  The policy is a set of thresholds measured on a few shapes; this makes a regression in it visible."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu

CALLS = 200
WINDOWS = 5

# candidates: name -> knobs; "default" (no knob) is what the library does by itself
MATVEC = {"default": {}, "unsplit": {"HQ_Q3_KSPLIT": 1}, "tiles32": {"HQ_Q3_TILE": 2}, "waves4": {"HQ_Q3_WAVES": 4},
          "steps2": {"HQ_Q3_STEPS": 2}}
LONG_K = {"default": {}, "unsplit": {"HQ_Q3_KSPLIT": 1}, "three_ranges": {"HQ_Q3_KSPLIT": 3}}
BATCH = {"default": {}, "gemm": {"HQ_Q3_SMALL_BATCH": 0}, "passes": {"HQ_Q3_ROW_BLOCKS": 0},
         "row_blocks": {"HQ_Q3_ROW_BLOCKS": 1}}
CASES = [
    (4096, 11008, 1, MATVEC),
    (4096, 11008, 4, BATCH),
    (4096, 11008, 8, BATCH),
    (4096, 11008, 16, BATCH),
    (4096, 4096, 1, MATVEC),
    (4096, 4096, 12, BATCH),
    (8192, 28672, 16, BATCH),
    (8192, 28672, 64, BATCH),
    (36864, 11008, 1, LONG_K),     # nine rounds of K, 172 column tiles: one workgroup per round
    (36864, 16384, 1, LONG_K),     # 256 tiles fill the compute units evenly: unsplit workgroups walk the rounds
]


def _time(lib, call, nbuf):
    import torch
    for i in range(10):
        call(i % nbuf)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(WINDOWS + 1)]
    k = 0
    ev[0].record()
    for w in range(WINDOWS):
        for _ in range(CALLS):
            call(k % nbuf)
            k += 1
        ev[w + 1].record()
    torch.cuda.synchronize()
    return min(ev[w].elapsed_time(ev[w + 1]) for w in range(WINDOWS)) * 1e3 / CALLS   # us per call, best window


@pytest.mark.parametrize("K,N,M,candidates", CASES, ids=["%dx%d_m%d" % c[:3] for c in CASES])
def test_default_plan_is_near_the_best(hq, K, N, M, candidates):
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    dev = "cuda:0"
    g = torch.Generator(device=dev)
    g.manual_seed(K + N + M)
    nbuf = max(2, int(560e6 // (3 * K // 32 * N * 4)) + 1)
    mats = [torch.randint(-2 ** 31, 2 ** 31 - 1, (3 * K // 32, N), dtype=torch.int32, device=dev, generator=g)
            for _ in range(nbuf)]
    s = torch.empty(N, device=dev).uniform_(0.005, 0.02, generator=g)
    z = s * torch.randint(3, 5, (N,), device=dev, generator=g).float()
    x = torch.randn(M, K, device=dev, generator=g)
    x = x[0].contiguous() if M == 1 else x.half()
    y = torch.empty(M, N, device=dev)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    px, ps, pz, py, pm = vp(x), vp(s), vp(z), vp(y), [vp(m) for m in mats]
    dt = 0 if M == 1 else 1

    def call(i):
        rc = lib.hq_q3_matvec(px, dt, pm[i], ps, pz, py, K, N, M, 0, stream)
        assert rc == 0, lib.hq_strerror(rc)

    times, plans = {}, {}
    try:
        for name, knobs in candidates.items():
            for k, v in knobs.items():
                assert lib.hq_set_tunable(k.encode(), v, 0) == 0
            plans[name] = lib.hq_q3_matvec_plan(K, N, M)
            times[name] = _time(lib, call, nbuf)
            for k in knobs:
                lib.hq_set_tunable(k.encode(), 0, 1)
    finally:
        for knobs in candidates.values():
            for k in knobs:
                lib.hq_set_tunable(k.encode(), 0, 1)
    best = min(times, key=times.get)
    print("K=%d N=%d M=%d: " % (K, N, M) + ", ".join("%s %.2f us (plan %d)" % (n, t, plans[n]) for n, t in times.items()))
    assert times["default"] <= 1.10 * times[best], (times, plans)
