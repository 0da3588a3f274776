"""The oracle's fused-producer chains (RMSNorm + quantize, SwiGLU product +
quantize) pinned against their closed forms in float64."""

import torch

from oracle import w8a8_oracle as O


def test_add_rmsnorm_closed_form_row():
    """Pins the oracle's rms_norm to the textbook formula in float64 on a tiny case."""
    x = torch.tensor([[3.0, -4.0, 0.0, 12.0, 1.0, -1.0, 2.0, 5.0]]).to(torch.bfloat16)
    w = torch.tensor([1.0, 0.5, 2.0, 1.0, 1.0, 1.0, 1.0, 0.25]).to(torch.bfloat16)
    _, _, _, y = O.add_rmsnorm_quantize_int8(x, w, 1e-5)
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean() + 1e-5) * w.double()
    torch.testing.assert_close(y.double(), want, rtol=2.0 ** -8, atol=0)


def test_silu_closed_form():
    """Pins the oracle's silu-product to x * sigmoid(x) in float64."""
    gate = torch.tensor([[-8.0, -1.0, -0.5, 0.0, 0.5, 1.0, 4.0, 20.0]]).to(torch.bfloat16)
    up = torch.tensor([[1.0, 2.0, -3.0, 7.0, 0.5, -1.0, 0.25, 1.0]]).to(torch.bfloat16)
    _, _, h = O.silu_mul_quantize_int8(gate, up)
    gd = gate.double()
    want = up.double() * gd / (1 + torch.exp(-gd))
    torch.testing.assert_close(h.double(), want, rtol=2.0 ** -7, atol=1e-30)


def test_quantizer_runs_on_the_rounded_activation():
    """The chain quantizes the bf16-rounded activation, row by row, with the same
    rule as the stand-alone per-token quantizer."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 64, generator=g).to(torch.bfloat16)
    r = torch.randn(4, 64, generator=g).to(torch.bfloat16)
    w = torch.ones(64).to(torch.bfloat16)
    xq, s, t, y = O.add_rmsnorm_quantize_int8(x, w, 1e-5, r)
    assert torch.equal(t, x + r)
    q2, s2 = O.int8_quantize_rows(y)
    assert torch.equal(xq, q2) and torch.equal(s, s2)
    assert xq.abs().max().item() == 127
