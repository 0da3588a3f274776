"""Decode attention kernel (GQA over the dense KV cache, split over the context)
against the oracle's float32 attention."""

import pytest
import torch

from oracle import decoder_oracle as D
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(b, h, hkv, s, max_len, positions, seed, nsplit):
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(seed)
    d = 128
    q = torch.randn(b, h, s, d, generator=g).to(torch.bfloat16)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    pos = torch.tensor(positions, dtype=torch.long)
    # what lies behind the newest position is not part of the contract: poison it
    kc[:, :, max(positions) + 1:] = float("nan")
    vc[:, :, max(positions) + 1:] = float("nan")
    got = _cabi.attn_decode(q.to(DEV), kc.to(DEV), vc.to(DEV), pos.to(DEV), nsplit=nsplit)
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[:, :, max(positions) + 1:] = 0
    vc2[:, :, max(positions) + 1:] = 0
    want = D.attn_cached(q, kc2, vc2, pos)
    assert got.shape == (b, s, h * d)
    assert_bf16_close(got, want, what=f"attn b={b} h={h}/{hkv} s={s} pos={positions} nsplit={nsplit}")


@pytest.mark.parametrize("nsplit", [0, 1, 3, 8])
def test_decode_step_config4_shape(nsplit):
    print(f"case nsplit={nsplit}", flush=True)
    _case(32, 16, 4, 1, 640, [513], seed=1, nsplit=nsplit)


@pytest.mark.parametrize("b,h,hkv,s,max_len,positions", [
    (2, 16, 4, 2, 64, [9, 10]),        # two new tokens, 8 query rows per KV head
    (3, 8, 8, 1, 40, [0]),             # first token: one visible key; n_rep 1
    (1, 4, 1, 2, 33, [15, 32]),        # n_rep 4, tile boundaries (keys 0..15 / 0..32)
    (5, 2, 1, 3, 100, [97, 98, 99]),   # n_rep 2 x 3 tokens = 6 rows -> the 8-row kernel
    (2, 16, 2, 1, 16, [15]),           # n_rep 8
])
def test_decode_small_shapes(b, h, hkv, s, max_len, positions):
    print(f"case b={b} h={h} hkv={hkv} s={s} max_len={max_len} pos={positions}", flush=True)
    for nsplit in (1, 4):
        _case(b, h, hkv, s, max_len, positions, seed=b + h + s, nsplit=nsplit)


def test_softmax_of_large_scores_is_stable():
    """scores of +-300 before the softmax: the running-max form must not overflow"""
    from astrai_amd.extension import _cabi
    b, h, hkv, s, max_len, d = 1, 4, 1, 1, 48, 128
    q = torch.full((b, h, s, d), 3.0, dtype=torch.bfloat16)
    kc = torch.zeros(b, hkv, max_len, d, dtype=torch.bfloat16)
    kc[:, :, 5] = 9.0
    kc[:, :, 37] = -9.0
    vc = torch.arange(max_len, dtype=torch.float32).reshape(1, 1, max_len, 1).expand(b, hkv, max_len, d).to(torch.bfloat16)
    pos = torch.tensor([47])
    got = _cabi.attn_decode(q.to(DEV), kc.to(DEV), vc.contiguous().to(DEV), pos.to(DEV), nsplit=4)
    want = D.attn_cached(q, kc, vc.contiguous(), pos)
    assert torch.isfinite(got).all()
    assert_bf16_close(got, want, what="large scores")
    assert abs(got.float().mean().item() - 5.0) < 0.1   # all weight on key 5


def test_attn_decode_rejects_unsupported():
    from astrai_amd.extension import _cabi
    q = torch.zeros(1, 4, 1, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim 128"):
        _cabi.attn_decode(q, kc, kc.clone(), torch.zeros(1, dtype=torch.long, device=DEV))
    q = torch.zeros(1, 16, 3, 128, dtype=torch.bfloat16, device=DEV)   # 4 x 3 = 12 query rows
    kc = torch.zeros(1, 4, 8, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="<= 8"):
        _cabi.attn_decode(q, kc, kc.clone(), torch.zeros(3, dtype=torch.long, device=DEV))


def test_quantized_output_is_the_quantizer_applied_to_the_bf16_output():
    from astrai_amd.extension import _cabi
    from oracle import w8a8_oracle as O
    g = torch.Generator().manual_seed(9)
    b, h, hkv, s, max_len, d = 4, 16, 4, 2, 80, 128
    q = torch.randn(b, h, s, d, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([70, 71], device=DEV)
    out = _cabi.attn_decode(q, kc, vc, pos, nsplit=4)
    oq, os_ = _cabi.attn_decode(q, kc, vc, pos, nsplit=4, quantized=True)
    wq, ws = O.int8_quantize_rows(out.cpu().reshape(b * s, h * d))
    assert torch.equal(oq.cpu(), wq) and torch.equal(os_.cpu(), ws)


def test_decode_random_sweep():
    """Thirty seeded random layouts: batch, grouping (n_rep * new tokens <= 8), context
    length, positions of the new tokens and split count all vary."""
    g = torch.Generator().manual_seed(2718)
    for i in range(30):
        n_rep = (1, 2, 4, 8)[int(torch.randint(0, 4, (1,), generator=g))]
        s = int(torch.randint(1, 8 // n_rep + 1, (1,), generator=g))
        hkv = int(torch.randint(1, 5, (1,), generator=g))
        b = int(torch.randint(1, 6, (1,), generator=g))
        max_len = int(torch.randint(s, 700, (1,), generator=g))
        first = int(torch.randint(0, max_len - s + 1, (1,), generator=g))
        positions = list(range(first, first + s))
        nsplit = (0, 1, 2, 5, 16)[i % 5]
        print(f"case {i}: b={b} h={hkv * n_rep}/{hkv} s={s} max_len={max_len} pos={positions} nsplit={nsplit}",
              flush=True)
        _case(b, hkv * n_rep, hkv, s, max_len, positions, seed=900 + i, nsplit=nsplit)
