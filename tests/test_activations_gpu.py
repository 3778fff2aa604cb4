"""Elementwise check of the epilogue activations at the bar of the reference's
tests/test_triton_activations.py:15-25 (silu, erf-gelu, tanh-gelu in fp32, atol = rtol = 1e-6
against torch.nn.functional).  The device functions are reached the way every caller reaches
them: as the epilogue of m_grouped_gemm, here with one expert whose weight is the identity
matrix, so that the product is x itself, exactly, and the output is act(x) as the epilogue
computes it.  The sigmoid divides through a 1-ulp reciprocal instruction and Phi(x) is a
rational approximation (Abramowitz & Stegun 7.1.26), so this is the test that holds those two
to the reference's bar; the derivatives go through act_bwd the same way."""
from functools import partial

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

ACTS = [
    ("silu", F.silu),
    ("gelu", F.gelu),
    ("approx_gelu", partial(F.gelu, approximate="tanh")),
]


def _through_the_epilogue(x, act):
    from moe_explore.hip_kernels.m_grouped_gemm import MGroupedGEMMParams, m_grouped_gemm
    rows, n = x.shape
    eye = torch.eye(n, device=x.device, dtype=x.dtype).unsqueeze(0)
    gi = torch.tensor([0, rows], dtype=torch.int32, device=x.device)
    return m_grouped_gemm(x, MGroupedGEMMParams(eye, gi, None, False, False, rows, 1, activation=act))


@pytest.mark.parametrize("name,torch_act", ACTS)
@pytest.mark.parametrize("shape,spread", [((16, 16), 1.0), ((256, 64), 1.0), ((128, 64), 4.0)])
def test_activation_fp32(name, torch_act, shape, spread):
    g = torch.Generator().manual_seed(shape[0] + len(name))
    x = (torch.randn(shape, generator=g) * spread).cuda()
    y = _through_the_epilogue(x, name)
    torch.testing.assert_close(y, torch_act(x), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("name,torch_act", [("swiglu", F.silu), ("geglu", F.gelu)])
def test_glu_activation_fp32(name, torch_act):
    """GLU epilogues pair neighbouring columns: even = gate, odd = up
    (functional/activation.py:19-20)."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn((64, 64), generator=g).cuda()
    y = _through_the_epilogue(x, name)
    want = torch_act(x[:, 0::2]) * x[:, 1::2]
    torch.testing.assert_close(y, want, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("name,torch_act", ACTS)
def test_activation_known_points_fp32(name, torch_act):
    """Zero, large arguments of both signs (no overflow to NaN, saturation to 0 and x) and the
    region around the minimum of the curves."""
    pts = torch.tensor([0.0, -0.0, 1e-8, -1e-8, 0.5, -0.5, 1.0, -1.0, -0.75, -1.2785, 3.0, -3.0, 6.0,
                        -6.0, 12.0, -12.0, 30.0, -30.0, 88.0, -88.0, 100.0, -100.0])
    x = torch.cat([pts, pts[:10]]).repeat(16, 1).contiguous().cuda()      # [16, 32]
    y = _through_the_epilogue(x, name)
    assert torch.isfinite(y).all()
    torch.testing.assert_close(y, torch_act(x), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("name,torch_act", ACTS)
def test_activation_gradient_fp32(name, torch_act):
    from moe_explore.hip_kernels.m_grouped_gemm import act_bwd
    g = torch.Generator().manual_seed(9)
    h = torch.randn((64, 48), generator=g).cuda()
    dy = torch.ones_like(h)
    dh, _, _ = act_bwd(h, dy, name)
    hr = h.clone().requires_grad_(True)
    torch_act(hr).sum().backward()
    torch.testing.assert_close(dh, hr.grad, atol=2e-6, rtol=2e-6)
