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
