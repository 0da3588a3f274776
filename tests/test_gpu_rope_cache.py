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


@pytest.mark.parametrize("b,s,h,hkv,d,max_len,k", [
    (32, 1, 16, 4, 128, 640, 2048),    # config-4 decode step
    (1, 1, 16, 4, 128, 64, 2048),      # one sequence
    (3, 7, 4, 2, 64, 32, 512),         # a short block of new tokens, 21 rows
    (4, 16, 2, 1, 16, 40, 256),        # 64 rows: the largest the fused kernel takes
    (5, 1, 8, 8, 32, 16, 1024),        # no grouping, 16-row workgroups of eight waves
    (2, 3, 96, 8, 128, 16, 256),       # a wide projection: 48-row workgroups
    (32, 512, 16, 4, 128, 640, 2048),  # config-4 prefill: the large-tile GEMM with the same epilogue
    (3, 700, 32, 8, 128, 1000, 256),   # ragged token count (2100 rows, last tile partly empty), two slabs
    (5, 413, 40, 4, 128, 500, 384),    # 2065 rows, N = 48 heads, three slabs
])
def test_projection_with_rotary_epilogue_equals_the_two_kernels(b, s, h, hkv, d, max_len, k):
    """The fused q|k|v projection + rotary + cache write against the int8 GEMM followed by
    the rotary / cache-write kernel: q and both caches bit for bit, untouched slots untouched."""
    from astrai_amd.extension import _cabi
    print(f"case b={b} s={s} h={h} hkv={hkv} d={d} max_len={max_len} k={k}", flush=True)
    g = torch.Generator().manual_seed(b * 1000 + s * 10 + d + k)
    n = (h + 2 * hkv) * d
    a = torch.randint(-127, 128, (b * s, k), generator=g, dtype=torch.int8).to(DEV)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(DEV)
    sa = (torch.rand(b * s, generator=g) * 0.01 + 0.001).to(DEV)
    sb = (torch.rand(n, generator=g) * 0.01 + 0.001).to(DEV)
    table = D.rotary_table(d, max_len, 10000.0)
    positions = torch.randperm(max_len, generator=g)[:s].sort().values
    freqs = table.index_select(0, positions).to(DEV)
    pos = positions.to(DEV)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    k1, v1, k2, v2 = kc.to(DEV), vc.to(DEV), kc.to(DEV), vc.to(DEV)
    qkv = _cabi.mm_int8(a, w, sa, sb).reshape(b, s, n)
    q_want = _cabi.rope_cache_write(qkv, freqs, pos, k1, v1, h, hkv, d)
    assert _cabi.mm_int8_rope_cache_supported(b * s, k, d, n, b, h, hkv, max_len)
    q_got = _cabi.mm_int8_rope_cache(a, w, sa, sb, freqs, pos, k2, v2, b, s, h, hkv, d)
    for name, got, want in (("q", q_got, q_want), ("k_cache", k2, k1), ("v_cache", v2, v1)):
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), name


def test_projection_with_rotary_epilogue_limits():
    from astrai_amd.extension import _cabi
    assert not _cabi.mm_int8_rope_cache_supported(65, 2048, 128)
    assert not _cabi.mm_int8_rope_cache_supported(8, 2048 + 128, 128)
    a = torch.zeros(65, 256, dtype=torch.int8, device=DEV)
    w = torch.zeros(4 * 16, 256, dtype=torch.int8, device=DEV)
    kc = torch.zeros(65, 1, 4, 16, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="at most 64"):
        _cabi.mm_int8_rope_cache(a, w, torch.ones(65, device=DEV), torch.ones(64, device=DEV),
                                 torch.zeros(1, 8, 2, device=DEV), torch.zeros(1, dtype=torch.long, device=DEV),
                                 kc, kc.clone(), 65, 1, 2, 1, 16)
    # a slot outside the cache writes nothing, q is still produced
    a = torch.ones(2, 256, dtype=torch.int8, device=DEV)
    kc = torch.zeros(2, 1, 4, 16, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    q = _cabi.mm_int8_rope_cache(a, torch.ones(64, 256, dtype=torch.int8, device=DEV), torch.ones(2, device=DEV),
                                 torch.ones(64, device=DEV), D.rotary_table(16, 8, 10000.0)[:1].to(DEV),
                                 torch.tensor([4], device=DEV), kc, vc, 2, 1, 2, 1, 16)
    torch.cuda.synchronize()
    assert q.abs().sum().item() > 0 and kc.abs().sum().item() == 0 and vc.abs().sum().item() == 0


def test_rope_cache_write_random_sweep():
    """Twenty seeded random layouts of the standalone rotary / cache-write kernel."""
    g = torch.Generator().manual_seed(5050)
    r = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for i in range(20):
        hkv = r(1, 5); h = hkv * (1, 2, 4, 8)[r(0, 4)]; d = 8 * r(1, 17)
        b, s = r(1, 6), r(1, 40)
        test_rope_cache_write_matches_tensor_ops(b, s, h, hkv, d, s + r(0, 50), bool(i % 3 == 0))
