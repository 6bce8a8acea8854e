"""The standalone rfft operator against `torch.fft.rfft` in float64 on the
zero-padded (optionally reversed) rows: rel err <= 1e-4 (the transform runs in
float32; 16-bit inputs are exact in float32)."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import extension as ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(3, 40), (2, 5, 1000), (4, 1024), (1, 16384), (2, 9000), (7, 1), (1, 33)])
@pytest.mark.parametrize("flip", [False, True])
def test_rfft_matches_torch(shape, flip, dtype):
    g = torch.Generator().manual_seed(shape[-1])
    x = torch.randn(*shape, generator=g).to(dtype)
    L = shape[-1]
    M = max(32, 1 << (L - 1).bit_length())
    y = ops.rfft(x.cuda(), flip)
    assert y.shape == shape[:-1] + (M + 1,) and y.dtype == torch.complex64
    src = x.double().flip(-1) if flip else x.double()
    want = torch.fft.rfft(src, n=2 * M)
    assert rel_err(torch.view_as_real(y), torch.view_as_real(want)) <= 1e-4


def test_rfft_limits():
    with pytest.raises(RuntimeError, match="16384"):
        ops.rfft(torch.zeros(1, 16385, device="cuda"))
    assert ops.rfft(torch.zeros(0, 64, device="cuda")).shape == (0, 65)
    # an impulse at lag 1: exp(-i pi k / M)
    x = torch.zeros(1, 64, device="cuda")
    x[0, 1] = 1.0
    k = torch.arange(65, device="cuda", dtype=torch.float64)
    want = torch.polar(torch.ones_like(k), -torch.pi * k / 64)
    assert rel_err(torch.view_as_real(ops.rfft(x)[0]), torch.view_as_real(want)) <= 1e-6
