"""Prefill attention kernel (causal GQA of a block of new tokens over the dense KV
cache) against the oracle's float32 attention."""

import pytest
import torch

from oracle import decoder_oracle as D

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _close(got, want, what):
    """The kernel rounds the probabilities to bf16 before P.V (as flash kernels do) and the
    output once more: elementwise |y - ref| <= 2e-2 |ref| + four bf16 ulps at rms(ref) (the
    largest of millions of near-zero outputs sits several deviations out)."""
    g, w = got.float().cpu(), want.float().cpu()
    assert g.shape == w.shape, (g.shape, w.shape)
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    rms = w.pow(2).mean().sqrt().item()
    err = (g - w).abs()
    bad = err > 2e-2 * w.abs() + 2.0 ** -6 * rms
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance; worst "
                           f"{err.max().item():.4g} at ref {w.flatten()[err.argmax()].item():.4g}, rms {rms:.4g}")


def _case(b, h, hkv, s, max_len, start, seed, scale=1.0):
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(seed)
    d = 128
    q = (torch.randn(b, h, s, d, generator=g) * scale).to(torch.bfloat16)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    pos = torch.arange(start, start + s, dtype=torch.long)
    last = start + s - 1
    # what lies behind the newest position is not part of the contract: poison it
    kc[:, :, last + 1:] = float("nan")
    vc[:, :, last + 1:] = float("nan")
    got = _cabi.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), pos.to(DEV))
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[:, :, last + 1:] = 0
    vc2[:, :, last + 1:] = 0
    want = D.attn_cached(q, kc2, vc2, pos)
    assert got.shape == (b, s, h * d) and got.dtype == torch.bfloat16
    _close(got, want, f"prefill b={b} h={h}/{hkv} s={s} start={start}")


@pytest.mark.parametrize("b,h,hkv,s,max_len,start", [
    (1, 4, 1, 1, 8, 0),        # one token, one key
    (2, 8, 2, 32, 32, 0),      # exactly one query block, cache exactly full
    (2, 8, 2, 33, 80, 0),      # one row into the second query block
    (1, 4, 1, 70, 96, 0),      # ragged: 3 query blocks, 2 key blocks
    (2, 8, 2, 64, 200, 40),    # chunked prefill: 40 cached tokens come first
    (1, 4, 1, 5, 300, 250),    # a short chunk deep into the context
    (3, 4, 2, 100, 128, 0),    # n_rep 2
    (1, 16, 2, 65, 130, 63),   # n_rep 8, block boundaries at 63 / 64
])
def test_prefill_small_shapes(b, h, hkv, s, max_len, start):
    print(f"case b={b} h={h} hkv={hkv} s={s} max_len={max_len} start={start}", flush=True)
    _case(b, h, hkv, s, max_len, start, seed=b + h + s + start)


def test_prefill_random_shape_sweep():
    """Thirty seeded random layouts: batch, grouping, chunk length, cache length and the
    chunk's start all vary, block boundaries (32 query rows, 64 keys) fall anywhere."""
    g = torch.Generator().manual_seed(31337)
    for i in range(30):
        n_rep = (2, 4, 8)[int(torch.randint(0, 3, (1,), generator=g))]
        hkv = int(torch.randint(1, 4, (1,), generator=g))
        b = int(torch.randint(1, 4, (1,), generator=g))
        s = int(torch.randint(1, 200, (1,), generator=g))
        start = int(torch.randint(0, 150, (1,), generator=g)) if i % 2 else 0
        max_len = start + s + int(torch.randint(0, 70, (1,), generator=g))
        print(f"case {i}: b={b} h={hkv * n_rep} hkv={hkv} s={s} max_len={max_len} start={start}", flush=True)
        _case(b, hkv * n_rep, hkv, s, max_len, start, seed=1000 + i)


def test_prefill_config4_shape():
    _case(2, 16, 4, 512, 640, 0, seed=4)


def test_prefill_sharp_softmax():
    """queries 4x larger: scores of +-45 before the softmax, nearly one-hot rows"""
    _case(1, 8, 2, 96, 96, 0, seed=9, scale=4.0)


def test_prefill_matches_decode_kernel_on_last_token():
    """the last token of a prefill is a decode step: both kernels agree on it"""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(77)
    b, h, hkv, s, max_len = 2, 16, 4, 150, 160
    q = torch.randn(b, h, s, 128, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.arange(s, device=DEV)
    full = _cabi.attn_prefill(q, kc, vc, pos)
    last = _cabi.attn_decode(q[:, :, -1:].contiguous(), kc, vc, pos[-1:])
    _close(full[:, -1:], last, "prefill vs decode on the last token")


def test_prefill_non_monotonic_positions():
    """positions need not increase: each token is masked by its own position"""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(5)
    b, h, hkv, s, max_len = 1, 4, 1, 40, 100
    q = torch.randn(b, h, s, 128, generator=g).to(torch.bfloat16)
    kc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, max_len, (s,), generator=g)
    got = _cabi.attn_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), pos.to(DEV))
    _close(got, D.attn_cached(q, kc, vc, pos), "scattered positions")


def test_attn_prefill_rejects_unsupported():
    from astrai_amd.extension import _cabi
    q = torch.zeros(1, 4, 3, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim 128"):
        _cabi.attn_prefill(q, kc, kc.clone(), torch.zeros(3, dtype=torch.long, device=DEV))
    q = torch.zeros(1, 4, 3, 128, dtype=torch.bfloat16, device=DEV)   # n_rep 1
    kc = torch.zeros(1, 4, 8, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="2, 4, 8"):
        _cabi.attn_prefill(q, kc, kc.clone(), torch.zeros(3, dtype=torch.long, device=DEV))
