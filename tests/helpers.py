"""Shared helpers for the parity tests."""

import torch


def assert_bf16_close(got: torch.Tensor, want: torch.Tensor, rel: float = 1e-2, what: str = ""):
    """The parity gate for scaled bf16 outputs: elementwise
    ``|y - ref| <= rel*|ref| + one bf16 ulp at rms(ref)`` and, on top, a normalised
    max error ``max|y-ref| / max|ref| <= rel``."""
    assert got.shape == want.shape, (got.shape, want.shape)
    g, w = got.float().cpu(), want.float().cpu()
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    rms = w.pow(2).mean().sqrt().item()
    ulp = 2.0 ** -8 * max(rms, 1e-30)
    err = (g - w).abs()
    bound = rel * w.abs() + ulp
    bad = err > bound
    assert not bad.any(), (
        f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance; "
        f"worst err {err.max().item():.4g} at ref {w.flatten()[err.argmax()].item():.4g}"
    )
    denom = w.abs().max().item()
    if denom > 0:
        assert err.max().item() / denom <= rel, f"{what}: normalised max error {err.max().item()/denom:.3g}"


def gpu_available() -> bool:
    return torch.cuda.is_available()
