"""Rotary embedding + KV-cache write kernel against the decoder oracle's tensor-op
chain (split, rotate in fp32, permute, index_copy)."""

import pytest
import torch

from oracle import decoder_oracle as D

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("b,s,h,hkv,d,max_len,strided", [
    (32, 1, 16, 4, 128, 640, False),     # config-4 decode step
    (2, 37, 16, 4, 128, 64, False),      # ragged prefill block
    (3, 5, 4, 2, 64, 16, True),          # qkv as a view into a wider buffer
    (1, 1, 1, 1, 8, 4, False),
])
def test_rope_cache_write_matches_tensor_ops(b, s, h, hkv, d, max_len, strided):
    from astrai_amd.extension import _cabi
    print(f"case b={b} s={s} h={h} hkv={hkv} d={d} max_len={max_len} strided={strided}", flush=True)
    g = torch.Generator().manual_seed(b * 100 + s + d)
    feat = (h + 2 * hkv) * d
    wide = torch.randn(b, s, feat + (16 if strided else 0), generator=g).to(torch.bfloat16)
    qkv = wide[..., :feat]
    table = D.rotary_table(d, max_len, 10000.0)
    positions = torch.randperm(max_len, generator=g)[:s].sort().values
    freqs = table.index_select(0, positions).unsqueeze(0)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    kd, vd = kc.to(DEV), vc.to(DEV)
    q_got = _cabi.rope_cache_write(wide.to(DEV)[..., :feat], freqs[0].to(DEV), positions.to(DEV), kd, vd, h, hkv, d)
    q_want = D.rope_cache_write(qkv, freqs, positions, kc, vc, h, hkv, d)
    assert q_got.shape == (b, h, s, d)
    for name, got, want in (("q", q_got, q_want), ("k_cache", kd, kc), ("v_cache", vd, vc)):
        assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16)), name


def test_rope_cache_write_skips_positions_outside_the_cache():
    from astrai_amd.extension import _cabi
    b, s, h, hkv, d, max_len = 2, 3, 2, 1, 16, 8
    qkv = torch.ones(b, s, (h + 2 * hkv) * d, dtype=torch.bfloat16, device=DEV)
    freqs = D.rotary_table(d, 16, 10000.0)[:s].to(DEV)
    kc = torch.zeros(b, hkv, max_len, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    pos = torch.tensor([1, 8, -1], device=DEV)   # 8 and -1 are outside [0, 8)
    _cabi.rope_cache_write(qkv, freqs, pos, kc, vc, h, hkv, d)
    torch.cuda.synchronize()
    assert vc[:, :, 1].abs().sum().item() > 0
    written = vc.abs().sum(dim=(0, 1, 3)) > 0
    assert written.tolist() == [False, True] + [False] * 6


def test_rope_cache_write_rejects_bad_arguments():
    from astrai_amd.extension import _cabi
    qkv = torch.zeros(1, 1, 4 * 12, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(1, 1, 4, 12, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        _cabi.rope_cache_write(qkv, torch.zeros(1, 6, 2, device=DEV), torch.zeros(1, dtype=torch.long, device=DEV),
                               kc, kc.clone(), 2, 1, 12)
    with pytest.raises(RuntimeError, match="features"):
        _cabi.rope_cache_write(qkv, torch.zeros(1, 8, 2, device=DEV), torch.zeros(1, dtype=torch.long, device=DEV),
                               kc, kc.clone(), 2, 1, 16)
