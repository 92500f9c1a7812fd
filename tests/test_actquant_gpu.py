"""Bit-exact parity of the per-token int8 activation quantisers with the CPU oracle (which
is pinned by the reference's own host loops), through the C ABI."""
import numpy as np
import pytest

from tests.test_oracle_cpu import _act_inputs

pytestmark = pytest.mark.gpu


def _dev(x):
    import torch
    return (x if isinstance(x, torch.Tensor) else torch.from_numpy(np.ascontiguousarray(x))).to("cuda:0")


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("tokens,hidden", [(64, 4096), (7, 200), (3, 8), (2, 13000), (16, 1001), (1, 1)])
def test_static_and_dynamic_bit_exact(hq, oracle, tokens, hidden, dtype):
    import torch
    x = _act_inputs(dtype, max(tokens, 2), hidden, tokens + hidden)[:tokens]
    dx = _dev(x)
    for azp in (None, 54):
        got = hq.static_scaled_int8_quant(dx, 0.1, azp)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), oracle.int8_quant_static(x, 0.1, azp)), azp
    for with_azp in (False, True):
        got, gs, gz = hq.dynamic_scaled_int8_quant(dx, with_azp)
        torch.cuda.synchronize()
        want, ws, wz = oracle.int8_quant_dynamic(x, with_azp)
        assert np.array_equal(gs.cpu().numpy(), ws)
        if with_azp:
            assert np.array_equal(gz.cpu().numpy(), wz)
        assert np.array_equal(got.cpu().numpy(), want), with_azp


@pytest.mark.parametrize("dtype,tokens,hidden", [("f16", 2100, 5137), ("bf16", 2100, 1001), ("f32", 2100, 8192),
                                                 ("f16", 2049, 8185), ("f32", 2200, 13), ("f16", 2051, 1),
                                                 ("f32", 2050, 777), ("f16", 300, 9000), ("f32", 5, 41001)])
def test_ragged_rows_wave_and_group_paths(hq, oracle, dtype, tokens, hidden):
    """Enough rows for the wave-per-row kernels, hidden sizes that leave every row unaligned, and rows beyond
    what a wave or a workgroup keeps in registers."""
    import torch
    x = _act_inputs(dtype, tokens, hidden, tokens * 3 + hidden)
    dx = _dev(x)
    for azp in (None, -7):
        got = hq.static_scaled_int8_quant(dx, 0.37, azp)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), oracle.int8_quant_static(x, 0.37, azp)), azp
    for with_azp in (False, True):
        got, gs, gz = hq.dynamic_scaled_int8_quant(dx, with_azp)
        torch.cuda.synchronize()
        want, ws, wz = oracle.int8_quant_dynamic(x, with_azp)
        assert np.array_equal(gs.cpu().numpy(), ws)
        if with_azp:
            assert np.array_equal(gz.cpu().numpy(), wz)
        assert np.array_equal(got.cpu().numpy(), want), with_azp


def test_fp16_subnormals_and_special_values(hq, oracle):
    """fp16 rows made of subnormal halves, of the largest halves, and rows that hold -0, infinities (static
    scale only) and isolated NaNs next to ordinary values (NaN is ignored by the reference's max / min and its quantised
    value is left out of the comparison): the fp16 kernels multiply the packed halves directly."""
    import torch
    rng = np.random.default_rng(77)
    rows = [rng.standard_normal(5137) * 3e-6,                       # all subnormal
            rng.standard_normal(5137) * 6e-5,                       # around the smallest normal half
            np.clip(rng.standard_normal(5137) * 2e4, -65504, 65504),  # up to the largest halves
            np.where(rng.random(5137) < 0.5, 5.96e-8, -5.96e-8),    # the smallest subnormal, both signs
            np.where(rng.random(5137) < 0.01, 0.0, rng.standard_normal(5137)) * np.where(rng.random(5137) < 0.5, 1, -1),
            rng.standard_normal(5137) + 3.0]
    x = np.stack(rows).astype(np.float16)
    x[4, 17] = np.float16(-0.0)
    x = np.concatenate([x, x[:, ::-1]], axis=0)
    dx = _dev(x)
    for scale in (1e-7, 3e-6, 0.5, 300.0):
        for azp in (None, 54):
            xs = x.copy()
            if azp is None:  # infinities saturate; with a dynamic scale or a zero point they are undefined
                xs[2, 5], xs[2, 4000] = np.float16(np.inf), np.float16(-np.inf)
            if azp is not None:  # int32 overflow of quotient + zero point is undefined in the reference as well
                with np.errstate(all="ignore"):
                    xs = np.where(np.abs(x.astype(np.float64) / scale) < 2.0e9, x, np.float16(0))
            got = hq.static_scaled_int8_quant(_dev(xs), scale, azp)
            torch.cuda.synchronize()
            assert np.array_equal(got.cpu().numpy(), oracle.int8_quant_static(xs, scale, azp)), (scale, azp)
    for with_azp in (False, True):
        got, gs, gz = hq.dynamic_scaled_int8_quant(dx, with_azp)
        torch.cuda.synchronize()
        want, ws, wz = oracle.int8_quant_dynamic(x, with_azp)
        assert np.array_equal(gs.cpu().numpy(), ws)
        if with_azp:
            assert np.array_equal(gz.cpu().numpy(), wz)
        assert np.array_equal(got.cpu().numpy(), want), with_azp
    # NaN elements: the row's scale comes from the others, and the others quantise as without the NaN
    y = x.copy()
    y[:, 100] = np.float16(np.nan)
    y[:, 4001] = np.float16(np.nan)
    keep = np.ones(y.shape[1], bool)
    keep[[100, 4001]] = False
    for with_azp in (False, True):
        got, gs, gz = hq.dynamic_scaled_int8_quant(_dev(y), with_azp)
        torch.cuda.synchronize()
        want, ws, wz = oracle.int8_quant_dynamic(y, with_azp)
        assert np.array_equal(gs.cpu().numpy(), ws)
        if with_azp:
            assert np.array_equal(gz.cpu().numpy(), wz)
        assert np.array_equal(got.cpu().numpy()[:, keep], want[:, keep]), with_azp


@pytest.mark.parametrize("scale", [0.1, 0.25, 0.3, 1.0 / 3.0, 7.0, 1e-3, 123.456, 2.0 ** -100, 2.0 ** 100, 2.0 ** -101,
                                   2.0 ** 101, 1e-40, 3e38, -0.5])
def test_static_division_ties_and_extreme_scales(hq, oracle, scale):
    """Inputs whose quotient by the scale sits on, or one float beside, a rounding tie or the saturation
    edges, and scales for which the reciprocal is not usable: the result must be that of the true
    division.  (NaN quotients are left out: converting them to an integer is undefined in the reference.)"""
    import torch
    s = np.float32(scale)
    k = np.arange(-140, 141, dtype=np.float64)
    with np.errstate(all="ignore"):
        ties = ((k + 0.5) * np.float64(s)).astype(np.float32)
        ints = (k * np.float64(s)).astype(np.float32)
        base = np.concatenate([ties, ints])
        beside = []  # one to six floats either side: the window in which product and quotient can round apart
        up, down = base, base
        for _ in range(6):
            up, down = np.nextafter(up, np.float32(np.inf)), np.nextafter(down, np.float32(-np.inf))
            beside += [up, down]
        x = np.concatenate([base] + beside + [
                            np.array([0.0, -0.0, np.inf, -np.inf, 3e38, -3e38, 1e-45, 1e30, -1e30], np.float32),
                            np.random.default_rng(3).standard_normal(3000).astype(np.float32) * np.float32(abs(scale)) * 60,
                            (np.arange(-2.0 ** 20, 2.0 ** 20, 2049.0) + 0.5) * np.float64(s),
                            (k + 0.5 + 2000000.0) * np.float64(s), (k + 0.5 - 2000000.0) * np.float64(s),
                            (k + 0.5 + 100.0) * np.float64(s), (k + 0.5 - 54.0) * np.float64(s)]).astype(np.float32)
    x = np.ascontiguousarray(np.resize(x, (4, x.size // 4)))
    dx = _dev(x)
    for azp in (None, 0, 54, -100, 2000000, -2000000):
        if azp is not None:  # int32 overflow of quotient + zero point is undefined in the reference as well
            with np.errstate(all="ignore"):
                x = np.where(np.abs(x.astype(np.float64) / np.float64(s)) < 2.0e9, x, np.float32(0))
            dx = _dev(x)
        got = hq.static_scaled_int8_quant(dx, float(s), azp)
        torch.cuda.synchronize()
        want = oracle.int8_quant_static(x, float(s), azp)
        bad = np.flatnonzero(got.cpu().numpy().ravel() != want.ravel())
        assert bad.size == 0, (scale, azp, x.ravel()[bad[:6]], got.cpu().numpy().ravel()[bad[:6]], want.ravel()[bad[:6]])


def test_unaligned_pointers(hq, oracle):
    """Views that start one element into an allocation: served element by element, same results."""
    import torch
    x = _act_inputs("f16", 9, 1001, 5)
    flat = torch.zeros(x.size + 8, dtype=torch.float16, device="cuda:0")
    dx = flat[1:1 + x.size].view(9, 1001)
    dx.copy_(_dev(x))
    assert dx.data_ptr() % 16 != 0
    assert np.array_equal(hq.static_scaled_int8_quant(dx, 0.1, 3).cpu().numpy(), oracle.int8_quant_static(x, 0.1, 3))
    got, gs, gz = hq.dynamic_scaled_int8_quant(dx, True)
    want, ws, wz = oracle.int8_quant_dynamic(x, True)
    assert np.array_equal(got.cpu().numpy(), want) and np.array_equal(gs.cpu().numpy(), ws)
    obuf = torch.zeros(x.size + 8, dtype=torch.int8, device="cuda:0")
    o = obuf[3:3 + x.size].view(9, 1001)
    got = hq.static_scaled_int8_quant(_dev(x), 0.1, None, out=o)
    torch.cuda.synchronize()
    assert np.array_equal(o.cpu().numpy(), oracle.int8_quant_static(x, 0.1, None))
    assert int(obuf[:3].abs().sum()) == 0 and int(obuf[3 + x.size:].abs().sum()) == 0


def test_reference_fixture(hq, oracle):
    """The reference main's own input: rand() % 1000 - 300, scale 0.1, azp 54 (main.cu:186-236)."""
    import torch
    rng = np.random.default_rng(123)
    x = rng.integers(-300, 700, size=(512, 4096)).astype(np.float16)
    dx = _dev(x)
    assert np.array_equal(hq.static_scaled_int8_quant(dx, 0.1).cpu().numpy(), oracle.int8_quant_static(x, 0.1))
    assert np.array_equal(hq.static_scaled_int8_quant(dx, 0.1, 54).cpu().numpy(), oracle.int8_quant_static(x, 0.1, 54))
    got, gs, gz = hq.dynamic_scaled_int8_quant(dx, True)
    torch.cuda.synchronize()
    want, ws, wz = oracle.int8_quant_dynamic(x, True)
    assert np.array_equal(got.cpu().numpy(), want) and np.array_equal(gs.cpu().numpy(), ws)
    assert np.array_equal(gz.cpu().numpy(), wz)


def test_empty_and_bad_arguments(hq):
    import torch
    x = torch.zeros((0, 16), dtype=torch.float16, device="cuda:0")
    assert hq.static_scaled_int8_quant(x, 0.1).numel() == 0
    with pytest.raises(ValueError):
        hq.static_scaled_int8_quant(torch.zeros((2, 2), dtype=torch.int32, device="cuda:0"), 0.1)


def test_full_size_error_bound(hq):
    """The reference's run size (4096 tokens of 5137) without the oracle: the dequantised values of the
    dynamic quantisers lie within half a step of the input, every row uses the full range, and the
    static quantiser agrees with the dynamic one when given a row's own scale."""
    import torch
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(11)
    x = (torch.randn(4096, 5137, device=dev, generator=g) * 3).half()
    xf = x.float()
    q, s, _ = hq.dynamic_scaled_int8_quant(x)
    assert np.array_equal(s.cpu().numpy(), xf.abs().amax(dim=1).cpu().numpy() / np.float32(127.0))  # true division
    assert float((q.float() * s[:, None] - xf).abs().div(s[:, None]).max()) <= 0.5 + 1e-3
    assert int(q.abs().amax(dim=1).min()) == 127
    qa, sa, za = hq.dynamic_scaled_int8_quant(x, True)
    assert float(((qa.float() - za[:, None].float()) * sa[:, None] - xf).abs().div(sa[:, None]).max()) <= 1.0 + 1e-3
    assert int(qa.amax(dim=1).min()) >= 126 and int(qa.amin(dim=1).max()) <= -127
    row = 1234
    qs = hq.static_scaled_int8_quant(x[row:row + 1].contiguous(), float(sa[row]), int(za[row]))
    assert torch.equal(qs[0], qa[row])


@pytest.mark.parametrize("dtype,code", [("f32", 0), ("f16", 1), ("bf16", 2)])
def test_vs_reference_device_kernels(hq, dtype, code):
    """The reference's own device kernels (src/quantVLLM-hip/main.cu), compiled into oracle/_ref, on the same
    device buffers: byte-for-byte equal, like the reference's own memcmp against its host loops."""
    import ctypes
    import torch
    from tests import oracle_api as oa
    ref = oa.load_ref_hip()
    if ref is None or not hasattr(ref, "ref_hip_int8_quant_static"):
        pytest.skip("oracle/_ref/libhecref_hip.so without the quantVLLM device kernels")
    tokens, hidden = 257, 5137
    x = _dev(_act_inputs(dtype, tokens, hidden, 17 + code))
    vp = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    for azp in (0, 54):
        want = torch.empty(tokens, hidden, dtype=torch.int8, device="cuda:0")
        ref.ref_hip_int8_quant_static(vp(x), code, vp(want), ctypes.c_long(tokens), hidden, ctypes.c_float(0.1), azp)
        torch.cuda.synchronize()
        assert torch.equal(hq.static_scaled_int8_quant(x, 0.1, azp if azp else None), want), azp
    for with_azp in (False, True):
        want = torch.empty(tokens, hidden, dtype=torch.int8, device="cuda:0")
        ws = torch.empty(tokens, device="cuda:0")
        wz = torch.empty(tokens, dtype=torch.int32, device="cuda:0") if with_azp else None
        ref.ref_hip_int8_quant_dynamic(vp(x), code, vp(want), vp(ws), vp(wz), ctypes.c_long(tokens), hidden)
        torch.cuda.synchronize()
        got, gs, gz = hq.dynamic_scaled_int8_quant(x, with_azp)
        assert torch.equal(gs, ws) and torch.equal(got, want), with_azp
        if with_azp:
            assert torch.equal(gz, wz)
