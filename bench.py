#!/usr/bin/env python3
"""Benchmark of the weight-only quantized-inference kernels on one MI355X.

Headline (the fields `metric`, `value`, `ms_per_step`, `roofline`): the GPTQ 3-bit matvec K=4096, N=11008
with fp32 activations - achieved HBM GB/s (algorithmic bytes / time per call) and microseconds per call,
weights rotated over more than 512 MB of distinct buffers so that no call is served from the 256 MB
Infinity Cache.  The same line carries, under `configs`, the other four benchmark configurations (NF4
dequantisation, LUT-GEMM, AQLM, batched 3-bit GEMM), each timed the same way with its own roofline object,
and under `other_kernels` the kernels of the neighbouring benchmarks (gemv fp16 / int8 / int4, mxfp4, the int8
activation quantisers, the 8-bit dynamic-map quantiser) at the reference programs' run sizes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--windows R] [--no-cpu] [--no-others] [--all]

A step is one library call.  After W warm-up calls, R windows of exactly K back-to-back calls are enqueued
with a HIP event between windows (on the stream the kernels are launched on; timing-only events without a
system-scope fence); `ms_per_step` is the MEDIAN
window divided by K, the fastest and slowest windows are reported next to it.  Prints ONE JSON line."""
import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, vendor figure
MFMA_F16_PEAK_TFLOPS = 2500.0

K, N = 4096, 11008
ROWS = 3 * K // 32
ALGO_BYTES = ROWS * N * 4 + 2 * N * 4 + K * 4 + N * 4   # weights + scale/zero + x + y = 17,056,768


def profile_traffic(name):
    """HBM bytes per launch of the dominant kernel of a configuration: FETCH_SIZE + WRITE_SIZE from two
    rocprofv3 --pmc runs, each scaled by what the same counter reads for a plain 256 MiB device copy, as
    recorded in profiles/<name>.txt.  None when the summary is missing."""
    try:
        text = open(os.path.join(ROOT, "profiles", name + ".txt")).read()
    except OSError:
        return None
    m = re.search(r"traffic \(fetched \+ written\) per launch: (\d+) bytes", text)
    return int(m.group(1)) if m else None


def _windows_for(steps, windows):
    if windows:
        return max(1, windows)
    # short windows are noisier: more of them (always an odd count, at least 11)
    return max(11, min(201, (20000 // max(steps, 1)) | 1))


_HIP = None


def _hip_runtime():
    """The HIP runtime this process already runs on (the copy torch loaded), for events created with
    hipEventDisableSystemFence: events that only measure time need no system-scope fence, whose cache
    write-back and invalidation would otherwise be charged to the first call of the next window (0.1 us per
    call in windows of 20 calls).  None if it cannot be found."""
    global _HIP
    if _HIP is None:
        _HIP = False
        try:
            with open("/proc/self/maps") as maps:
                paths = {line.split()[-1] for line in maps if "libamdhip64.so" in line}
            if len(paths) == 1:
                lib = ctypes.CDLL(paths.pop())
                lib.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
                lib.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
                lib.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
                lib.hipEventDestroy.argtypes = [ctypes.c_void_p]
                _HIP = lib
        except (OSError, AttributeError):
            _HIP = False
    return _HIP or None


HIP_EVENT_DISABLE_SYSTEM_FENCE = 0x20000000


def _time_windows(fn, n_buffers, steps, warmup, windows):
    """R windows of `steps` back-to-back calls on torch's current stream (the stream the kernels are
    enqueued on), a HIP event between windows, one synchronisation at the end.  Returns the sorted list of
    seconds per window."""
    import torch
    for i in range(warmup):
        fn(i % n_buffers)
    torch.cuda.synchronize()
    hip = _hip_runtime()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    raw = []
    if hip is not None:
        for _ in range(windows + 1):
            e = ctypes.c_void_p()
            if hip.hipEventCreateWithFlags(ctypes.byref(e), HIP_EVENT_DISABLE_SYSTEM_FENCE) != 0:
                for made in raw:
                    hip.hipEventDestroy(made)
                raw, hip = [], None
                break
            raw.append(e)
    if hip is None:
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(windows + 1)]
        record = lambda j: ev[j].record()
    else:
        def record(j):
            if hip.hipEventRecord(raw[j], stream) != 0:
                raise RuntimeError("hipEventRecord failed")
    k = 0
    record(0)
    for w in range(windows):
        for _ in range(steps):
            fn(k % n_buffers)
            k += 1
        record(w + 1)
    torch.cuda.synchronize()
    if hip is None:
        return sorted(ev[w].elapsed_time(ev[w + 1]) * 1e-3 for w in range(windows))
    secs = []
    ms = ctypes.c_float()
    for w in range(windows):
        if hip.hipEventElapsedTime(ctypes.byref(ms), raw[w], raw[w + 1]) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        secs.append(ms.value * 1e-3)
    for e in raw:
        hip.hipEventDestroy(e)
    return sorted(secs)


def _summary(secs, steps):
    """median / fastest / slowest window as microseconds per call"""
    med = secs[len(secs) // 2]
    return med / steps * 1e6, secs[0] / steps * 1e6, secs[-1] / steps * 1e6


def measure_device():
    """What this box delivers to the simplest kernels (hq_probe_*): a pure read and a copy of 512 MiB (more
    than the 256 MB Infinity Cache), and independent 16-byte reads at random entries of a 1 MB table (a
    code-book lookup without the arithmetic: the rate of L2 requests)."""
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    n = 512 << 20
    src = [torch.empty(n, dtype=torch.uint8, device=dev).random_() for _ in range(2)]
    dst = torch.empty(n, dtype=torch.uint8, device=dev)
    ps = [ctypes.c_void_p(t.data_ptr()) for t in src]
    pd = ctypes.c_void_p(dst.data_ptr())

    def check(rc):
        if rc:
            raise RuntimeError(lib.hq_strerror(rc).decode())

    out = {}
    secs = _time_windows(lambda i: check(lib.hq_probe_stream(0, ps[i], pd, n, stream)), 2, 10, 4, 11)
    out["hbm_read_measured_GBps"] = round(n / (secs[len(secs) // 2] / 10) / 1e9, 1)
    secs = _time_windows(lambda i: check(lib.hq_probe_stream(1, ps[i], pd, n, stream)), 2, 10, 4, 11)
    out["hbm_copy_measured_GBps"] = round(2 * n / (secs[len(secs) // 2] / 10) / 1e9, 1)
    out["hbm_probe"] = "hq_probe_stream over 512 MiB, two source buffers alternating; copy counts bytes read + written"
    del src, dst
    table = torch.empty(1 << 20, dtype=torch.uint8, device=dev).random_()
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    want = 1 << 24
    cnt = lib.hq_probe_gather16_count(want)
    pt, pk = ctypes.c_void_p(table.data_ptr()), ctypes.c_void_p(sink.data_ptr())
    secs = _time_windows(lambda i: check(lib.hq_probe_gather16(pt, 1 << 20, want, pk, stream)), 1, 20, 5, 11)
    out["l2_gather16_measured_Greq_s"] = round(cnt / (secs[len(secs) // 2] / 20) / 1e9, 1)
    out["l2_gather_probe"] = ("hq_probe_gather16: %d independent 16-byte reads per launch at random entries of a "
                              "1 MB table, eight in flight per lane" % cnt)
    return out


# the 16 lanes of each of the two passes a half wave's 128-bit LDS read is served in (measured on gfx950)
_PASS_A = [0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27]
PASS_OF = [0 if l in _PASS_A else 1 for l in range(32)]
PASS_RANK = [(_PASS_A.index(l) if l in _PASS_A else [m for m in range(32) if m not in _PASS_A].index(l)) for l in range(32)]


def lds_patterns():
    """(name, width in bits, write, byte offset per lane) of the LDS access patterns hq_probe_lds is run on:
    patterns whose conflicts are known, and the operand layouts of the matvec kernels (lane = 16 * quarter + c)."""
    lanes = range(64)
    c = lambda l: l & 15
    kb = lambda l: l >> 4
    piece = lambda row, quarter, half: 16 * row + 512 * quarter + 176 * half   # q3.hip dig_piece
    xs = lambda l: (l >> 3) & 3
    xkb = lambda l: ((l >> 2) & 1) * 2 + (l >> 5)
    pats = [
        ("read b32, consecutive words", 32, 0, [4 * l for l in lanes]),
        ("read b64, consecutive", 64, 0, [8 * l for l in lanes]),
        ("read b128, consecutive", 128, 0, [16 * l for l in lanes]),
        ("read b32, 8 bytes apart (two lanes of a pass per bank)", 32, 0, [8 * l for l in lanes]),
        ("read b32, 128 bytes apart (a pass in one bank)", 32, 0, [(128 * l) % 8192 for l in lanes]),
        ("read b128, 256 bytes apart (a pass in one bank group)", 128, 0, [(256 * l) % 8192 for l in lanes]),
        ("write b32, consecutive words", 32, 1, [4 * l for l in lanes]),
        ("write b128, consecutive", 128, 1, [16 * l for l in lanes]),
        ("read b128, passes as measured (lanes 0-3, 12-15, 20-27 | 4-11, 16-19, 28-31 per half wave): the lanes "
         "of a pass at 16 consecutive pieces, every pass 256 bytes further", 128, 0,
         [16 * PASS_RANK[l & 31] + 256 * PASS_OF[l & 31] + 512 * (l >> 5) for l in lanes]),
        ("read b128, lanes 16-31 and 48-63 rotated by eight pieces: free of conflicts if a pass were 16 consecutive "
         "lanes, two-way with the passes as measured", 128, 0,
         [16 * ((l + 8 * ((l >> 4) & 1)) & 15) + 256 * (l >> 4) for l in lanes]),
        ("read b128, 3-bit matvec digit operand in rows of 144 bytes (the former layout)", 128, 0,
         [min(c(l), 8) * 144 + kb(l) * 32 for l in lanes]),
        ("read b128, 3-bit matvec digit operand, first half (q3.hip)", 128, 0,
         [piece(c(l) if c(l) < 8 else 8 + (kb(l) & 1), kb(l), 0) for l in lanes]),
        ("read b128, 3-bit matvec digit operand, second half, step 3", 128, 0,
         [3 * 1888 + piece(c(l) if c(l) < 8 else 8 + (kb(l) & 1), kb(l), 1) for l in lanes]),
        ("write b32, 3-bit matvec digit staging, row 0 even elements", 32, 1,
         [xs(l) * 1888 + piece(0, 2 * (xkb(l) & 1), xkb(l) >> 1) + 4 * (l & 3) for l in lanes]),
        ("write b32, 3-bit matvec digit staging, row 1 odd elements", 32, 1,
         [xs(l) * 1888 + piece(1, 2 * (xkb(l) & 1) + 1, xkb(l) >> 1) + 4 * (l & 3) for l in lanes]),
        ("read b128, LUT digit operand of a three-plane set, 32-byte rows (the former layout)", 128, 0,
         [(c(l) & 3) * 32 + 16 * (kb(l) & 1) if (c(l) >> 2) == (kb(l) >> 1) else 512 for l in lanes]),
        ("read b128, LUT digit operand of a three-plane set (lut.hip)", 128, 0,
         [16 * (c(l) & 3) + 336 * (kb(l) & 1) if (c(l) >> 2) == (kb(l) >> 1) else 144 for l in lanes]),
        ("read b128, small-batch kernel's sixteen operand rows (q3_block.hip)", 128, 0,
         [16 * c(l) + 256 * (kb(l) & 1) + 512 * (kb(l) >> 1) for l in lanes]),
    ]
    return pats


def lds_probe(repeats=4096, launches=20):
    """hq_probe_lds on every pattern of lds_patterns(), `launches` launches each, in that order (a profiler's
    dispatches can be matched by order); microseconds per launch."""
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"repeats_per_lane": repeats, "launches": launches, "patterns": []}
    for name, width, write, offs in lds_patterns():
        table = torch.tensor(offs, dtype=torch.int32, device=dev)

        def call(_i):
            rc = lib.hq_probe_lds(ctypes.c_void_p(table.data_ptr()), width, write, repeats,
                                  ctypes.c_void_p(sink.data_ptr()), stream)
            if rc:
                raise RuntimeError("hq_probe_lds: " + lib.hq_strerror(rc).decode())
        secs = _time_windows(call, 1, launches, 2, 3)
        out["patterns"].append({"name": name, "width": width, "write": write,
                                "us_per_launch": round(_summary(secs, launches)[0], 2)})
    return out


def bench_q3(steps, warmup, windows, hot=False):
    import torch
    from hecbench_amd import _lib
    dev = torch.device("cuda:0")
    lib = _lib.load()
    n_buf = 1 if hot else 34           # 34 x 16.9 MB = 575 MB of distinct weights
    g = torch.Generator(device=dev)
    g.manual_seed(1234)
    # any 32-bit pattern is a valid string of 3-bit codes: uniform random words = uniform codes
    mats = [torch.randint(-2 ** 31, 2 ** 31 - 1, (ROWS, N), dtype=torch.int32, device=dev, generator=g)
            for _ in range(n_buf)]
    scales = torch.empty(N, device=dev).uniform_(0.005, 0.02, generator=g)
    zeros = scales * torch.randint(3, 5, (N,), device=dev, generator=g).float()
    x = torch.randn(K, device=dev, generator=g)
    y = torch.empty(N, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    px, ps, pz, py = (ctypes.c_void_p(t.data_ptr()) for t in (x, scales, zeros, y))
    pm = [ctypes.c_void_p(m.data_ptr()) for m in mats]

    def call(i):
        rc = lib.hq_q3_matvec(px, 0, pm[i], ps, pz, py, K, N, 1, 0, stream)
        if rc:
            raise RuntimeError(lib.hq_strerror(rc).decode())

    secs = _time_windows(call, n_buf, steps, warmup, windows)
    return secs, dict(x=x, scales=scales, zeros=zeros, mat0=mats[0], y=y, call=call, mats=mats,
                      ptrs=(px, ps, pz, py, pm))


def graph_replay_q3(state_args, calls=34, replays=200):
    """The headline call recorded into a HIP graph (`calls` back-to-back calls on rotated weight buffers, captured
    once) and replayed: microseconds per call of the replays, i.e. with the launch pitch of a graph instead of
    `calls` separate launches."""
    import torch
    from hecbench_amd import _lib
    lib = _lib.load()
    px, ps, pz, py, pm = state_args
    side = torch.cuda.Stream()
    # the workspace of the capture stream exists before the capture (this shape needs none; kept for the rule)
    lib.hq_reserve_workspace(ctypes.c_void_p(side.cuda_stream), K, N)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for i in range(calls):
            rc = lib.hq_q3_matvec(px, 0, pm[i % len(pm)], ps, pz, py, K, N, 1, 0, st)
            if rc:
                raise RuntimeError(lib.hq_strerror(rc).decode())
    for _ in range(5):
        graph.replay()
    torch.cuda.synchronize()
    windows = 11
    per = max(1, replays // windows)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(windows + 1)]
    ev[0].record()
    for w in range(windows):
        for _ in range(per):
            graph.replay()
        ev[w + 1].record()
    torch.cuda.synchronize()
    secs = sorted(ev[w].elapsed_time(ev[w + 1]) * 1e-3 for w in range(windows))
    return secs[windows // 2] / (per * calls) * 1e6


def _roofline_hbm(algo_bytes, us, profile):
    gbs = algo_bytes / us / 1e3
    return {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": profile_traffic(profile)}


def bench_configs(steps, warmup, windows, device=None):
    """Configurations 0, 2, 3 and 4 of the benchmark: microseconds per call (median window), algorithmic GB/s
    and the roofline object of each; inputs rotated over more than 512 MB so that every call reads HBM."""
    import torch
    from hecbench_amd import _lib
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(99)
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}

    def vp(t):
        return ctypes.c_void_p(t.data_ptr())

    def check(rc):
        if rc:
            raise RuntimeError(lib.hq_strerror(rc).decode())

    def entry(name, workload, algo_bytes, secs, st, profile, **extra):
        us, lo, hi = _summary(secs, st)
        e = {"workload": workload, "us_per_call": round(us, 3), "us_per_call_min": round(lo, 3),
             "us_per_call_max": round(hi, 3), "steps": st, "windows": len(secs),
             "algorithmic_bytes_per_call": algo_bytes, "GBps": round(algo_bytes / us / 1e3, 1),
             "roofline": _roofline_hbm(algo_bytes, us, profile)}
        e.update(extra)
        out[name] = e
        return us

    # config 0: NF4 dequant 4096x4096, blocksize 64 (rotate 14 x 43 MB)
    n = 4096 * 4096
    nb = 14
    packed = [torch.randint(0, 256, (n // 2,), dtype=torch.uint8, device=dev, generator=g) for _ in range(nb)]
    absmax = [torch.empty(n // 64, device=dev).uniform_(0.5, 2.0, generator=g) for _ in range(nb)]
    outs = [torch.empty(n, dtype=torch.float16, device=dev) for _ in range(nb)]
    args = [(vp(packed[i]), vp(absmax[i]), vp(outs[i])) for i in range(nb)]
    secs = _time_windows(lambda i: check(lib.hq_dequant_nf4(args[i][0], args[i][1], args[i][2], n, 64, 0, stream)),
                         nb, steps, warmup, windows)
    entry("0_nf4_dequant_4096x4096", "NF4 dequant 4096x4096, blocksize 64, fp16 out, 14 rotated buffer sets (602 MB)",
          n // 2 + n // 64 * 4 + 64 + n * 2, secs, steps, "nf4_dequant_4096x4096", dtype="f32 multiply -> f16")
    del packed, absmax, outs
    # config 2: LUT-GEMM K=4096 N=16384 q=3 G=128 (rotate 20 x 29 MB)
    Kl, Nl = 4096, 16384
    nb = 20
    bW = [torch.randint(-2 ** 31, 2 ** 31 - 1, (Kl // 32, 3, Nl), dtype=torch.int32, device=dev, generator=g)
          for _ in range(nb)]
    alpha = [(torch.randn(Kl // 128, 3, Nl, device=dev, generator=g) * 0.02).abs().half() for _ in range(nb)]
    qb = torch.zeros(Kl // 128, Nl, dtype=torch.float16, device=dev)
    xl = torch.randn(Kl, device=dev, generator=g).half()
    yl = torch.empty(Nl, dtype=torch.float16, device=dev)
    args = [(vp(bW[i]), vp(alpha[i])) for i in range(nb)]
    pq, px, py = vp(qb), vp(xl), vp(yl)
    secs = _time_windows(lambda i: check(lib.hq_lut_gemv(args[i][0], args[i][1], pq, px, py, Kl, Nl, 3, 128, stream)),
                         nb, steps, warmup, windows)
    entry("2_lut_gemv_4096x16384_q3", "LUT-GEMM K=4096 N=16384, 3 bit planes, group 128, 20 rotated weight sets (566 MB)",
          Kl // 32 * 3 * Nl * 4 + Kl // 128 * 3 * Nl * 2 + Kl // 128 * Nl * 2 + Kl * 2 + Nl * 2, secs, steps,
          "lut_gemv_4096x16384_q3", dtype="f16 in, exact integer sums, f32 alpha, f16 out")
    del bW, alpha
    # config 3: AQLM 4096x4096 (rotate 128 x 4 MB of codes; the 1 MB code book is shared)
    Ma, Ka = 4096, 4096
    nb = 128
    codes = [torch.randint(-32768, 32768, (Ma, Ka // 8), dtype=torch.int16, device=dev, generator=g)
             for _ in range(nb)]
    cb = (torch.randn(65536, 8, device=dev, generator=g) * 0.05).half()
    sc = torch.empty(Ma, device=dev).uniform_(0.5, 1.5, generator=g).half()
    xa = torch.randn(Ka, device=dev, generator=g).half()
    ya = torch.empty(Ma, dtype=torch.float16, device=dev)
    args = [vp(c) for c in codes]
    pcb, psc, pxa, pya = vp(cb), vp(sc), vp(xa), vp(ya)
    sizes = (ctypes.c_int * 4)(Ma, 0, 0, 0)
    secs = _time_windows(lambda i: check(lib.hq_aqlm_matvec(args[i], pcb, psc, pxa, pya, Ma, Ka, sizes, 65536, stream)),
                         nb, steps, warmup, windows)
    us = entry("3_aqlm_4096x4096", "AQLM 1x16 M=4096 K=4096, one code book, 128 rotated code sets (537 MB)",
               Ma * Ka // 8 * 2 + 65536 * 16 + 3 * Ka * 2, secs, steps, "aqlm_matvec_4096x4096",
               dtype="f16 in, f32 sums, f16 out")
    out["3_aqlm_4096x4096"]["gather_GBps"] = round(Ma * Ka // 8 * 16 / us / 1e3, 1)   # 16-byte code-book gathers (L2)
    # what bounds this kernel: one L2 request per 16-byte code-book entry; the peak is the rate the same box
    # delivers to a kernel that does nothing but such reads from a table of the same size
    peak = (device or {}).get("l2_gather16_measured_Greq_s")
    greq = Ma * Ka // 8 / us / 1e3
    out["3_aqlm_4096x4096"]["roofline_l2_requests"] = {
        "bound": "l2_requests", "achieved": round(greq, 1), "peak": peak, "unit": "G 16-byte gathers/s",
        "frac": None if not peak else round(greq / peak, 4), "traffic": None}
    del codes
    # config 4: batched GPTQ 3-bit GEMM M=64 K=8192 N=28672 (rotate 7 x 88 MB)
    Mg, Kg, Ng = 64, 8192, 28672
    nb = 7
    mats = [torch.randint(-2 ** 31, 2 ** 31 - 1, (3 * Kg // 32, Ng), dtype=torch.int32, device=dev, generator=g)
            for _ in range(nb)]
    sg = torch.empty(Ng, device=dev).uniform_(0.005, 0.02, generator=g)
    zg = sg * torch.randint(3, 5, (Ng,), device=dev, generator=g).float()
    Ag = torch.randn(Mg, Kg, device=dev, generator=g).half()
    og = torch.empty(Mg, Ng, device=dev)
    pA, psg, pzg, pog = vp(Ag), vp(sg), vp(zg), vp(og)
    pm = [vp(m) for m in mats]
    st = max(10, min(steps, 500))
    secs = _time_windows(lambda i: check(lib.hq_q3_matvec(pA, 1, pm[i], psg, pzg, pog, Kg, Ng, Mg, 0, stream)),
                         nb, st, min(warmup, 50), windows)
    fl = 2.0 * Mg * Kg * Ng
    us = entry("4_q3_gemm_64x8192x28672", "batched GPTQ 3-bit GEMM M=64 K=8192 N=28672, fp16 activations, 7 rotated "
               "weight buffers (617 MB); one call = activation pre-pass + main kernel",
               3 * Kg // 32 * Ng * 4 + 2 * Ng * 4 + Mg * Kg * 2 + Mg * Ng * 4, secs, st, "q3_gemm_64x8192x28672",
               dtype="f16 MFMA, f32 accumulate")
    tf = fl / us / 1e6
    out["4_q3_gemm_64x8192x28672"]["roofline_mfma"] = {"bound": "mfma", "achieved": round(tf, 1),
                                                       "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                                       "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None}
    del mats, Ag, og
    # the headline shape at batches 4 and 8 (extension: one pass over the weights for all rows, 34 rotated buffers)
    Ks, Ns = K, N
    nb = 34
    mats = [torch.randint(-2 ** 31, 2 ** 31 - 1, (3 * Ks // 32, Ns), dtype=torch.int32, device=dev, generator=g)
            for _ in range(nb)]
    ss = torch.empty(Ns, device=dev).uniform_(0.005, 0.02, generator=g)
    zs = ss * torch.randint(3, 5, (Ns,), device=dev, generator=g).float()
    pm = [vp(m) for m in mats]
    for Ms in (4, 8):
        As = torch.randn(Ms, Ks, device=dev, generator=g).half()
        os_ = torch.empty(Ms, Ns, device=dev)
        pA, pss, pzs, pos = vp(As), vp(ss), vp(zs), vp(os_)
        plan = lib.hq_q3_matvec_plan(Ks, Ns, Ms)
        secs = _time_windows(lambda i: check(lib.hq_q3_matvec(pA, 1, pm[i], pss, pzs, pos, Ks, Ns, Ms, 0, stream)),
                             nb, steps, warmup, windows)
        entry("1_q3_matvec_4096x11008_batch%d" % Ms,
              "GPTQ 3-bit K=4096 N=11008, %d fp16 activation rows in one call, 34 rotated weight buffers (575 MB)" % Ms,
              3 * Ks // 32 * Ns * 4 + 2 * Ns * 4 + Ms * Ks * 2 + Ms * Ns * 4, secs, steps, "q3_batch%d_4096x11008" % Ms,
              dtype="fp6 x fp8 MFMA, exact integer sums, f32 out",
              kernel={2: "batched GEMM", 3: "four rows per pass"}.get(plan, str(plan)))
    del mats
    return out


def cpu_baseline_q3(state, budget_s=12.0):
    """The oracle's serial restatement of the reference fp32 kernel on one host core,
    on weight buffer 0; doubles as the correctness check of the timed GPU buffers."""
    import numpy as np
    import torch
    from tests import oracle_api as oa
    from tests.tol import rel_err
    o = oa.load_oracle()
    mat = state["mat0"].cpu().numpy()
    x = state["x"].cpu().numpy()
    s = state["scales"].cpu().numpy()
    z = state["zeros"].cpu().numpy()
    state["call"](0)
    torch.cuda.synchronize()
    got = state["y"].cpu().numpy()
    t0 = time.perf_counter()
    ref = o.q3_matvec_f32(x, mat, s, z)
    one = time.perf_counter() - t0
    err = rel_err(got, ref)
    reps = max(3, int(budget_s / max(one, 1e-3)))
    t0 = time.perf_counter()
    for _ in range(reps):
        o.q3_matvec_f32(x, mat, s, z)
    per = (time.perf_counter() - t0) / reps
    # the same loops spread over the host cores with OpenMP (columns partitioned, same results)
    _, threads = o.q3_matvec_f32_omp(x, mat, s, z)
    oreps = max(3, int(0.5 * budget_s / max(one / max(threads, 1), 1e-3)))
    t0 = time.perf_counter()
    for _ in range(oreps):
        o.q3_matvec_f32_omp(x, mat, s, z)
    oper = (time.perf_counter() - t0) / oreps
    return {"value": round(ALGO_BYTES / per / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "us_per_call": round(per * 1e6, 1),
            "sample": f"{reps} serial calls of the oracle's fp32 restatement (4096x11008, one weight buffer)",
            "openmp": {"value": round(ALGO_BYTES / oper / 1e9, 3), "unit": "GB/s", "cores": threads,
                       "us_per_call": round(oper * 1e6, 1), "sample": f"{oreps} calls"},
            "gpu_vs_oracle_max_rel_err": err}


def bench_others(steps, warmup, windows):
    """The kernels of the neighbouring benchmarks (gemv, mxfp4, quantVLLM, quantBnB): microseconds per call
    (median window) and algorithmic GB/s."""
    import numpy as np
    import torch
    import hecbench_amd as hq
    from hecbench_amd import _lib
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(199)
    out = {}
    # raw C-ABI calls with prepared arguments: the Python wrappers cost as much as the short kernels take
    lib = _lib.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def vp(t):
        return ctypes.c_void_p(t.data_ptr())

    def check(rc):
        if rc:
            raise RuntimeError(lib.hq_strerror(rc).decode())

    def _time_loop(fn, n_buffers, st, wu):
        secs = _time_windows(fn, n_buffers, st, wu, windows)
        return secs[len(secs) // 2]

    # next rows: dense / int8 / int4 gemv at the reference's run size 16384 x 16384 (the weight buffers are
    # rotated so that at least 512 MB of distinct data passes between two uses of a buffer) and mxfp4
    # quantise-dequantise of 4096 x 4096 fp16 elements (rotate 16 x 67 MB)
    ng = 16384
    vg = torch.rand(ng, device=dev, generator=g).half()
    rg = torch.empty(ng, dtype=torch.float16, device=dev)
    st = max(50, steps // 8)
    for name, nbuf, make, call, bytes_per in (
            ("gemv_fp16_16384", 2, lambda: torch.rand(ng, ng, device=dev, generator=g).half(),
             lambda m: hq.gemv_fp16(m, vg, out=rg), 2.0),
            ("gemv_int8_16384", 3, lambda: torch.randint(-128, 128, (ng, ng), dtype=torch.int8, device=dev, generator=g),
             lambda m: hq.gemv_int8(m, vg, 0.0625, 0.01, out=rg), 1.0),
            ("gemv_int4_16384", 5, lambda: torch.randint(0, 256, (ng, ng // 2), dtype=torch.uint8, device=dev, generator=g),
             lambda m: hq.gemv_int4(m, vg, 0.0625, 0.01, out=rg), 0.5)):
        bufs = [make() for _ in range(nbuf)]
        secs = _time_loop(lambda i: call(bufs[i]), nbuf, st, 5)
        b = bytes_per * ng * ng + 4.0 * ng
        out[name] = {"us": secs / st * 1e6, "GBps": b * st / secs / 1e9, "frac_hbm": b * st / secs / 1e9 / HBM_PEAK_GBS}
        del bufs
    nm = 4096 * 4096
    nb = 16
    src = [torch.randn(nm, device=dev, generator=g).half() for _ in range(nb)]
    dst = [torch.empty(nm, dtype=torch.float16, device=dev) for _ in range(nb)]
    secs = _time_loop(lambda i: hq.mxfp4_qdq(src[i], out=dst[i]), nb, steps, warmup)
    b = 4.0 * nm
    out["mxfp4_qdq_4096x4096_f16"] = {"us": secs / steps * 1e6, "GBps": b * steps / secs / 1e9,
                                      "frac_hbm": b * steps / secs / 1e9 / HBM_PEAK_GBS}
    del src, dst
    # quantVLLM at its default run size: 4096 tokens of 5137 fp16 activations -> int8 (rotate 12 x 63 MB)
    tk, hd = 4096, 5137
    nb = 12
    xs = [(torch.randint(-300, 700, (tk, hd), device=dev, generator=g)).half() for _ in range(nb)]
    qo = [torch.empty(tk, hd, dtype=torch.int8, device=dev) for _ in range(nb)]
    scl = torch.empty(tk, device=dev)
    azp = torch.empty(tk, dtype=torch.int32, device=dev)
    args = [(vp(xs[i]), vp(qo[i])) for i in range(nb)]
    psc, paz = vp(scl), vp(azp)
    b = 3.0 * tk * hd
    for name, call in (
            ("int8_quant_static_4096x5137_f16",
             lambda i: check(lib.hq_int8_quant_static(args[i][0], 1, args[i][1], tk, hd, ctypes.c_float(0.1), 0, 0, stream))),
            ("int8_quant_static_azp_4096x5137_f16",
             lambda i: check(lib.hq_int8_quant_static(args[i][0], 1, args[i][1], tk, hd, ctypes.c_float(0.1), 1, 3, stream))),
            ("int8_quant_dynamic_4096x5137_f16",
             lambda i: check(lib.hq_int8_quant_dynamic(args[i][0], 1, args[i][1], psc, None, tk, hd, stream))),
            ("int8_quant_dynamic_azp_4096x5137_f16",
             lambda i: check(lib.hq_int8_quant_dynamic(args[i][0], 1, args[i][1], psc, paz, tk, hd, stream)))):
        secs = _time_loop(call, nb, steps, warmup)
        out[name] = {"us": secs / steps * 1e6, "GBps": b * steps / secs / 1e9,
                     "frac_hbm": b * steps / secs / 1e9 / HBM_PEAK_GBS}
    del xs, qo
    # the quantBnB benchmark's own kernel at its default size: 16,777,216 floats -> 8-bit codes (rotate 8 x 84 MB)
    nq = 16777216
    nb = 8
    code = hq.dynamic_map().to(dev)  # the table the reference quantises with
    As = [torch.randn(nq, device=dev, generator=g) for _ in range(nb)]
    qs = [torch.empty(nq, dtype=torch.uint8, device=dev) for _ in range(nb)]
    secs = _time_loop(lambda i: hq.quantize_dynamic8(code, As[i], out=qs[i]), nb, st, 5)
    b = 5.0 * nq + 1024
    out["quantize_dynamic8_16777216"] = {"us": secs / st * 1e6, "GBps": b * st / secs / 1e9,
                                         "frac_hbm": b * st / secs / 1e9 / HBM_PEAK_GBS}
    for name, e in out.items():
        algo = int(round(e["GBps"] * e["us"] * 1e3))
        e["algorithmic_bytes_per_call"] = algo
        e["roofline"] = _roofline_hbm(algo, e["us"], name)
        e["us"], e["GBps"], e["frac_hbm"] = round(e["us"], 3), round(e["GBps"], 1), round(e["frac_hbm"], 4)
    return out


def cpu_configs():
    """Serial and OpenMP times of the oracle's restatements for configurations 0, 2, 3 and 4 (bounded samples,
    scaled to the full problem where a sample is used; about five seconds in all).  Reported next to the GPU
    numbers, never a target."""
    import numpy as np
    from tests import oracle_api as oa
    o = oa.load_oracle()
    threads = max(1, min(o.max_threads(), os.cpu_count() or 1))

    def timed(fn, reps):
        """(median, best) seconds of `reps` single calls"""
        t = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            t.append(time.perf_counter() - t0)
        t.sort()
        return t[len(t) // 2], t[0]

    jobs = {}
    packed, absmax = oa.make_nf4_problem(0, 4096 * 4096, 64)
    jobs["0_nf4_dequant_4096x4096"] = (lambda: o.dequant_4bit(packed, absmax, 4096 * 4096, 64), 3, 1, "3 full calls")
    bW, alpha, qb, x = oa.make_lut_problem(0, 4096, 2048, 3, 128)
    jobs["2_lut_gemv_4096x16384_q3"] = (lambda: o.lut_gemv_f64(bW, alpha, qb, x, 128), 3, 8,
                                        "3 calls on 2048 of 16384 columns, scaled x8")
    codes, cb, sc, xa = oa.make_aqlm_problem(0, 4096, 4096)
    jobs["3_aqlm_4096x4096"] = (lambda: o.aqlm_matvec(codes, cb, sc, xa, (4096, 0, 0, 0), 65536), 3, 1, "3 full calls")
    qc, scales, zeros, A = oa.make_q3_problem(0, 8192, 1024, np.float16, batch=4)
    mat = o.q3_pack(qc)
    jobs["4_q3_gemm_64x8192x28672"] = (lambda: o.q3_gemm(A, mat, scales, zeros), 3, 16 * 28,
                                       "3 calls on 4 of 64 rows x 1024 of 28672 columns, scaled x448")
    out = {}
    for name, (fn, reps, scale, sample) in jobs.items():
        o.set_threads(1)
        s_med, s_best = timed(fn, reps)
        o.set_threads(threads)
        try:
            p_med, p_best = timed(fn, reps)
        finally:
            o.set_threads(1)
        out[name] = {"cpu_serial": {"us": round(s_med * scale * 1e6, 1), "us_best": round(s_best * scale * 1e6, 1), "cores": 1,
                                    "kind": "port", "sample": sample + " (median; best beside it)"},
                     "cpu_openmp": {"us": round(p_med * scale * 1e6, 1), "us_best": round(p_best * scale * 1e6, 1),
                                    "cores": threads, "kind": "port", "sample": sample + " (median; best beside it)"}}
    return out


def cpu_others():
    """Serial CPU times of the oracle for the other configurations (one host core; bounded samples, scaled to
    the full problem where a sample is used).  Reported next to the GPU numbers, never a target."""
    import numpy as np
    from tests import oracle_api as oa
    o = oa.load_oracle()
    out = {}

    def timed(fn, reps=1):
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    packed, absmax = oa.make_nf4_problem(0, 4096 * 4096, 64)
    out["nf4_dequant_4096x4096"] = {"cpu_us": timed(lambda: o.dequant_4bit(packed, absmax, 4096 * 4096, 64), 3) * 1e6,
                                    "sample": "3 full calls"}
    bW, alpha, qb, x = oa.make_lut_problem(0, 4096, 2048, 3, 128)
    out["lut_gemv_4096x16384_q3"] = {"cpu_us": timed(lambda: o.lut_gemv_f64(bW, alpha, qb, x, 128)) * 8 * 1e6,
                                     "sample": "2048 of 16384 columns, scaled x8"}
    codes, cb, sc, xa = oa.make_aqlm_problem(0, 4096, 4096)
    out["aqlm_4096x4096"] = {"cpu_us": timed(lambda: o.aqlm_matvec(codes, cb, sc, xa, (4096, 0, 0, 0), 65536), 3) * 1e6,
                             "sample": "3 full calls"}
    codes, scales, zeros, A = oa.make_q3_problem(0, 8192, 1024, np.float16, batch=4)
    mat = o.q3_pack(codes)
    out["q3_gemm_64x8192x28672"] = {"cpu_us": timed(lambda: o.q3_gemm(A, mat, scales, zeros)) * 16 * 28 * 1e6,
                                    "sample": "4 of 64 rows x 1024 of 28672 columns, scaled x448"}
    rng = np.random.default_rng(0)
    m8 = rng.integers(-128, 128, (1024, 16384)).astype(np.int8)
    v = rng.uniform(0, 1, 16384).astype(np.float16)
    out["gemv_int8_16384"] = {"cpu_us": timed(lambda: o.gemv(m8, 1, v, 0.0625, 0.01)) * 16 * 1e6,
                              "sample": "1024 of 16384 rows, scaled x16"}
    bits = rng.standard_normal(4096 * 4096).astype(np.float16).view(np.uint16)
    out["mxfp4_qdq_4096x4096_f16"] = {"cpu_us": timed(lambda: o.mxfp4_qdq(bits, False)) * 1e6, "sample": "1 full call"}
    xa8 = rng.integers(-300, 700, (512, 5137)).astype(np.float16)
    o.int8_quant_static(xa8[:1], 0.1)  # the oracle builds its fp16 conversion table on first use
    out["int8_quant_static_4096x5137_f16"] = {"cpu_us": timed(lambda: o.int8_quant_static(xa8, 0.1)) * 8 * 1e6,
                                              "sample": "512 of 4096 tokens, scaled x8"}
    out["int8_quant_dynamic_azp_4096x5137_f16"] = {"cpu_us": timed(lambda: o.int8_quant_dynamic(xa8, True)) * 8 * 1e6,
                                                   "sample": "512 of 4096 tokens, scaled x8"}
    # 8-bit quantiser: the reference's own host function where oracle/_ref holds it, else the oracle's restatement
    A = rng.standard_normal(1 << 21).astype(np.float32)
    q = np.zeros(A.size, np.uint8)
    ref = oa.load_ref_cpu()
    if ref is not None:
        fn = lambda: ref.ref_dquantize_n(A.ctypes.data_as(ctypes.c_void_p), q.ctypes.data_as(ctypes.c_void_p),
                                         ctypes.c_long(A.size))
        kind = "reference"
    else:
        code = o.dynamic_map()
        fn = lambda: o.quantize_dynamic8(code, A)
        kind = "port"
    out["quantize_dynamic8_16777216"] = {"cpu_us": timed(fn) * 8 * 1e6, "kind": kind,
                                         "sample": "2,097,152 of 16,777,216 elements, scaled x8"}
    omp = reference_quantbnb_omp()
    if omp is not None:
        out["quantize_dynamic8_16777216"]["reference_omp"] = omp
    return out


def quantbnb_host_only():
    """The build's own quantBnB driver run host-only (its verification loops spread over the host cores with
    OpenMP, no GPU call): what the benchmark's -omp variant measures with OMP_TARGET_OFFLOAD=DISABLED."""
    import subprocess
    exe = os.path.join(ROOT, "hecbench_amd", "bench", "quantBnB")
    if not os.path.exists(exe):
        return None
    try:
        r = subprocess.run([exe, "16777216", "3", "--host-only"], capture_output=True, text=True, timeout=120)
    except (subprocess.TimeoutExpired, OSError):
        return None
    m = re.search(r"kQuantize kernel with block size \d+: ([0-9.]+) \(us\)\n(PASS|FAIL)\n\s+\(host only: OpenMP loop on "
                  r"(\d+) threads; one thread: ([0-9.]+) us\)", r.stdout)
    if not m:
        return None
    return {"cpu_openmp": {"us": round(float(m.group(1)), 1), "cores": int(m.group(3)), "kind": "port",
                           "sample": "quantBnB 16777216 3 --host-only (the driver's own host loop)",
                           "verdict": m.group(2)},
            "cpu_serial": {"us": round(float(m.group(4)), 1), "cores": 1, "kind": "port",
                           "sample": "the same loop on one thread, one pass"}}


def reference_quantbnb_omp():
    """The reference's own quantBnB-omp program (compiled into oracle/_ref where the HeCBench tree was mounted),
    run host-only with OMP_TARGET_OFFLOAD=DISABLED in a child process; returns what it prints, or None."""
    import re
    import subprocess
    from tests import oracle_api as oa
    if not os.path.exists(oa.REF_CPU_SO):
        return None
    code = ("import ctypes,sys; lib=ctypes.CDLL(sys.argv[1]); "
            "argv=(ctypes.c_char_p*3)(b'main', b'16777216', b'3'); sys.exit(lib.ref_quantbnb_omp_main(3, argv))")
    env = dict(os.environ, OMP_TARGET_OFFLOAD="DISABLED")
    try:
        r = subprocess.run([sys.executable, "-c", code, oa.REF_CPU_SO], capture_output=True, text=True, env=env,
                           timeout=120)
    except subprocess.TimeoutExpired:
        return None
    m = re.search(r"Average execution time of kQuantize kernel with block size \d+: ([0-9.]+) \(us\)", r.stdout)
    if not m:
        return None
    return {"us": float(m.group(1)), "cores": int(os.environ.get("OMP_NUM_THREADS") or os.cpu_count()),
            "kind": "reference",
            "sample": "quantBnB-omp main, 16,777,216 elements x 3, OMP_TARGET_OFFLOAD=DISABLED",
            "verdict": "PASS" if "PASS" in r.stdout else "FAIL"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--windows", type=int, default=0,
                    help="timed windows of --steps calls (default: 11, more when --steps is small)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="time the headline configuration only")
    ap.add_argument("--no-others", action="store_true",
                    help="skip the kernels of the neighbouring benchmarks (gemv, mxfp4, quantVLLM, quantBnB)")
    ap.add_argument("--all", action="store_true",
                    help="also time the CPU restatements of the other configurations and kernels")
    ap.add_argument("--no-hot", action="store_true", help="skip the hot-cache (single buffer) timing")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 20 plain device copies of 256 MiB (reference point for rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--lds-probe", action="store_true",
                    help="run only hq_probe_lds, every pattern 20 times (LDS accesses whose bank conflicts are "
                         "known, for reading rocprofv3's SQ_LDS_BANK_CONFLICT against them), and print their times")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path has no collective and every box here has one GPU; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.steps < 1 or args.warmup < 0:
        print("--steps must be >= 1 and --warmup >= 0", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU path exists for the product kernels)", file=sys.stderr)
        sys.exit(2)
    import hecbench_amd as hq
    hq.init()
    info = hq.device_info()
    windows = _windows_for(args.steps, args.windows)

    if args.lds_probe:
        print(json.dumps(lds_probe()))
        return

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_()
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    secs, state = bench_q3(args.steps, args.warmup, windows)
    us, us_min, us_max = _summary(secs, args.steps)
    gbs = ALGO_BYTES / us / 1e3
    graph_us = None if args.no_hot else graph_replay_q3(state["ptrs"])
    hot_us = None if args.no_hot else _summary(bench_q3(args.steps, args.warmup, windows, hot=True)[0], args.steps)[0]
    result = {
        "metric": "achieved HBM GB/s: GPTQ-3bit matvec 4096x11008 (algorithmic bytes / time per call)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us * 1e-3, 6), "us_per_call": round(us, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "GPTQ 3-bit matvec K=4096 N=11008 batch 1, fp32 x, weights rotated over 34 "
                               "distinct 16.9 MB buffers (575 MB)", "algorithmic_bytes_per_call": ALGO_BYTES},
        "windows": windows, "ms_per_step_min": round(us_min * 1e-3, 6), "ms_per_step_max": round(us_max * 1e-3, 6),
        "timing": f"median of {windows} windows of {args.steps} back-to-back calls, HIP events on the launch stream "
                  f"({'created with hipEventDisableSystemFence' if _hip_runtime() else 'torch events'})",
        "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "effective_fp16_weight_GBps": round(K * N * 2 / us / 1e3, 1),
        "hot_cache_us_per_call": None if hot_us is None else round(hot_us, 3),
        "graph_replay_us_per_call": None if graph_us is None else round(graph_us, 3),
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": profile_traffic("q3_matvec_4096x11008")},
        "device": info,
    }
    result["device"] = dict(info, **measure_device())
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_q3(state)
    del state
    if not args.no_configs:
        # the other four benchmark configurations: a few thousand calls each at most
        st = max(1, min(args.steps, 1000))
        result["configs"] = bench_configs(st, min(args.warmup, 100), _windows_for(st, args.windows), result["device"])
        if not args.no_cpu:
            for name, legs in cpu_configs().items():
                if name in result["configs"]:
                    result["configs"][name].update(legs)
    if not args.no_others:
        # the kernels of the neighbouring benchmarks (gemv, mxfp4, quantVLLM, quantBnB), shorter loops
        st = max(20, min(args.steps // 4, 500))
        result["other_kernels"] = bench_others(st, 20, _windows_for(st, args.windows) if args.steps < 200 else 11)
    if not args.no_others and not args.no_cpu:
        legs = quantbnb_host_only()
        if legs:
            result["other_kernels"]["quantize_dynamic8_16777216"].update(legs)
    if args.all and not args.no_others:
        if not args.no_cpu:
            cpu = cpu_others()
            for name, c in cpu.items():
                tgt = result["other_kernels"].get(name)
                if tgt is None and not args.no_configs:
                    tgt = next((v for k, v in result["configs"].items() if k[2:] == name), None)
                if tgt is None:
                    continue
                if "cpu_serial" not in tgt:
                    tgt["cpu_serial"] = {"us": round(c["cpu_us"], 1), "cores": 1, "kind": c.get("kind", "port"),
                                         "sample": c["sample"]}
                if "reference_omp" in c:
                    tgt["cpu_reference_omp"] = c["reference_omp"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
