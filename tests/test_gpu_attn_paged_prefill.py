"""Ragged paged prefill attention (packed queries, token-granular pool, the reference's
attn_paged_prefill interface) against the oracle."""

import pytest
import torch

from oracle import decoder_oracle as D

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _close(got, want, what):
    """Same bound as the dense prefill kernel's test: probabilities and output are rounded to
    bf16: |y - ref| <= 2e-2 |ref| + four bf16 ulps at rms(ref)."""
    g, w = got.float().cpu(), want.float().cpu()
    assert g.shape == w.shape, (g.shape, w.shape)
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    rms = w.pow(2).mean().sqrt().item()
    err = (g - w).abs()
    bad = err > 2e-2 * w.abs() + 2.0 ** -6 * rms
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance; worst {err.max().item():.4g}"


def _setup(h, hkv, kv_lens, q_lens, max_ctx, pool, seed, holes=False):
    g = torch.Generator().manual_seed(seed)
    d, b = 128, len(kv_lens)
    n_req = b + 3
    q = torch.randn(sum(q_lens), h, d, generator=g).to(torch.bfloat16)
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    rows = torch.randperm(n_req, generator=g)[:b].int()
    table = torch.full((n_req, max_ctx), -1, dtype=torch.int32)
    perm = torch.randperm(pool, generator=g)
    nxt = 0
    for i in range(b):
        for j in range(kv_lens[i]):
            table[rows[i], j] = int(perm[nxt]); nxt += 1
        if holes and kv_lens[i] > 4:
            table[rows[i], 2] = -1
    unused = perm[nxt:]
    k_pool[unused] = float("nan")   # slots no live position maps to must not be read
    v_pool[unused] = float("nan")
    kvp = torch.tensor([0] + torch.tensor(kv_lens).cumsum(0).tolist(), dtype=torch.int32)
    return q, k_pool, v_pool, table, rows, kvp


def _run(args, q_lens, causal=True, mask=None):
    from astrai_amd.extension import _cabi
    qo, tb, ti = _cabi.paged_prefill_schedule(q_lens, DEV)
    dev = [t.to(DEV) for t in args]
    got = _cabi.attn_paged_prefill(*dev, qo, tb, ti, causal_offset=0 if causal else -1,
                                   mask=None if mask is None else mask.to(DEV))
    want = D.attn_paged_prefill(*args, qo.cpu(), causal=causal, mask=mask)
    return got, want


@pytest.mark.parametrize("h,hkv,kv_lens,q_lens", [
    (4, 1, [1], [1]),                              # one token
    (8, 2, [64, 64], [64, 64]),                    # whole tiles, whole prompts
    (8, 2, [65, 33, 200], [65, 33, 100]),          # ragged; the third continues a cached context
    (16, 4, [512, 17, 300, 64], [512, 17, 1, 64]),  # a decode-like single row among prompts
    (4, 2, [130, 70], [129, 3]),                   # n_rep 2
    (16, 2, [90], [90]),                           # n_rep 8
])
def test_paged_prefill_ragged(h, hkv, kv_lens, q_lens):
    print(f"case h={h}/{hkv} kv={kv_lens} q={q_lens}", flush=True)
    args = _setup(h, hkv, kv_lens, q_lens, max(kv_lens) + 5, sum(kv_lens) + 11, seed=h + sum(kv_lens))
    got, want = _run(args, q_lens)
    assert got.shape == (sum(q_lens), h, 128) and got.dtype == torch.bfloat16
    _close(got, want, f"paged prefill kv={kv_lens} q={q_lens}")


def test_paged_prefill_without_causal_mask_and_with_padding_slots():
    args = _setup(8, 2, [100, 40], [30, 40], 128, 200, seed=5, holes=True)
    got, want = _run(args, [30, 40], causal=False)
    _close(got, want, "non-causal, holes")
    got, want = _run(args, [30, 40], causal=True)
    _close(got, want, "causal, holes")


def test_paged_prefill_rows_without_keys_give_zeros():
    """an empty sequence, and more query rows than keys: the rows that see nothing are zero"""
    args = _setup(4, 1, [0, 3], [2, 5], 16, 32, seed=9)
    got, want = _run(args, [2, 5])
    _close(got, want, "rows without keys")
    assert torch.equal(got[:2].cpu(), torch.zeros(2, 4, 128, dtype=torch.bfloat16))
    assert torch.equal(got[2:4].cpu(), torch.zeros(2, 4, 128, dtype=torch.bfloat16))  # rows 0,1 of 5 see keys < 0


def test_paged_prefill_equals_dense_kernel_on_the_same_cache():
    """a pool that is the dense cache re-indexed, equal lengths: both kernels, same numbers"""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(21)
    b, h, hkv, n = 3, 16, 4, 150
    q = torch.randn(b, h, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    dense = _cabi.attn_prefill(q, kc, vc, torch.arange(n, device=DEV))            # [b, n, h*128]
    k_pool = kc.permute(0, 2, 1, 3).reshape(b * n, hkv, 128).contiguous()
    v_pool = vc.permute(0, 2, 1, 3).reshape(b * n, hkv, 128).contiguous()
    table = torch.arange(b * n, dtype=torch.int32, device=DEV).reshape(b, n)
    rows = torch.arange(b, dtype=torch.int32, device=DEV)
    kvp = (torch.arange(b + 1, device=DEV) * n).int()
    qo, tb, ti = _cabi.paged_prefill_schedule([n] * b, DEV)
    qp = q.permute(0, 2, 1, 3).reshape(b * n, h, 128).contiguous()
    paged = _cabi.attn_paged_prefill(qp, k_pool, v_pool, table, rows, kvp, qo, tb, ti, causal_offset=0)
    assert torch.equal(paged.reshape(b, n, -1), dense)


def test_paged_prefill_rejects_what_it_does_not_do():
    from astrai_amd.extension import _cabi
    args = [t.to(DEV) for t in _setup(4, 1, [3], [3], 8, 8, seed=2)]
    qo, tb, ti = _cabi.paged_prefill_schedule([3], DEV)
    with pytest.raises(RuntimeError, match="int32"):
        _cabi.attn_paged_prefill(*args, qo.long(), tb, ti)
    # the reference's mask checks (csrc/kernels/attention/entry_utils.cuh:326-346)
    ok = torch.ones(1, 1, 3, 3, dtype=torch.bool, device=DEV)
    for bad, msg in ((ok.float(), "bool"), (ok.cpu(), "CUDA"), (ok[0], "2D or 4D"),
                     (ok.expand(2, 1, 3, 3), "batch"), (ok.expand(1, 3, 3, 3), "head"),
                     (ok[:, :, :0], "q_len"), (ok[..., :0], "kv_len")):
        with pytest.raises(RuntimeError, match=msg):
            _cabi.attn_paged_prefill(*args, qo, tb, ti, mask=bad)


def _random_mask(shape, seed, keep=0.7):
    g = torch.Generator().manual_seed(seed)
    return torch.rand(shape, generator=g) < keep


@pytest.mark.parametrize("kind", ["2d", "4d_rows", "4d_heads", "4d_one_row"])
@pytest.mark.parametrize("causal", [True, False])
def test_paged_prefill_with_a_mask_tensor(kind, causal):
    """The reference's optional mask: [batch, kv] or [batch, 1 | H, rows, kv], True = attend,
    rows counted inside each sequence, 'and'-ed with the causal range."""
    h, hkv = 8, 2
    kv_lens, q_lens = [150, 70, 40], [150, 30, 40]
    width = max(kv_lens) + 5
    args = _setup(h, hkv, kv_lens, q_lens, width, sum(kv_lens) + 11, seed=17, holes=True)
    shape = {"2d": (3, width), "4d_rows": (3, 1, max(q_lens), width),
             "4d_heads": (3, h, max(q_lens), width), "4d_one_row": (3, h, 1, width)}[kind]
    mask = _random_mask(shape, seed=len(kind))
    if mask.dim() == 4 and mask.size(2) > 1:
        mask[1, :, 3] = False            # a row that sees nothing: zeros
        mask[0, :, :, :64] = False       # sequence 0: the whole first key block hidden from every row
    print(f"case {kind} causal={causal}", flush=True)
    got, want = _run(args, q_lens, causal=causal, mask=mask)
    _close(got, want, f"mask {kind} causal={causal}")
    if mask.dim() == 4 and mask.size(2) > 1:
        assert got[150 + 3].abs().sum() == 0


def test_paged_prefill_mask_smaller_than_the_sequences_and_strided():
    """Rows and positions that the mask does not hold are not attended; the mask may be a
    strided view (only its innermost stride has to be 1) or a batch broadcast."""
    h, hkv = 4, 2
    kv_lens, q_lens = [100, 90], [60, 90]
    args = _setup(h, hkv, kv_lens, q_lens, 128, 220, seed=23)
    big = _random_mask((2, 1, 80, 256), seed=5, keep=0.8)
    mask = big[:, :, :, 10:90]                 # 80 rows, 80 positions, row stride 256
    got, want = _run(args, q_lens, causal=True, mask=mask)
    _close(got, want, "narrow strided mask")
    assert got[60 + 80:].abs().sum() == 0      # rows 80.. of sequence 1: no row in the mask
    one = _random_mask((1, 128), seed=6).expand(2, 128)    # batch stride 0
    got, want = _run(args, q_lens, causal=False, mask=one)
    _close(got, want, "batch-broadcast mask")
    # an all-True mask is the unmasked kernel's result
    full = torch.ones(2, 128, dtype=torch.bool)
    got, _ = _run(args, q_lens, causal=True, mask=full)
    plain, _ = _run(args, q_lens, causal=True)
    _close(got, plain, "all-True mask")


def test_paged_prefill_random_sweep():
    """Twenty seeded random batches: request counts, grouping, cached prefix lengths and new
    token counts all vary; every third batch is non-causal, every fourth has padding slots."""
    g = torch.Generator().manual_seed(4242)
    for i in range(20):
        n_rep = (2, 4, 8)[int(torch.randint(0, 3, (1,), generator=g))]
        hkv = int(torch.randint(1, 4, (1,), generator=g))
        b = int(torch.randint(1, 5, (1,), generator=g))
        q_lens = [int(torch.randint(1, 150, (1,), generator=g)) for _ in range(b)]
        kv_lens = [ql + (int(torch.randint(0, 120, (1,), generator=g)) if j % 2 else 0)
                   for j, ql in enumerate(q_lens)]
        causal = i % 3 != 2
        print(f"case {i}: h={hkv * n_rep}/{hkv} kv={kv_lens} q={q_lens} causal={causal}", flush=True)
        args = _setup(hkv * n_rep, hkv, kv_lens, q_lens, max(kv_lens) + 3, sum(kv_lens) + 7,
                      seed=500 + i, holes=(i % 4 == 3))
        got, want = _run(args, q_lens, causal=causal)
        _close(got, want, f"sweep {i}")
        if i % 2:
            shape = [(b, max(kv_lens) + 3), (b, 1, max(q_lens), max(kv_lens) + 3),
                     (b, hkv * n_rep, max(q_lens), max(kv_lens))][(i // 2) % 3]
            got, want = _run(args, q_lens, causal=causal, mask=_random_mask(shape, seed=900 + i, keep=0.5))
            _close(got, want, f"sweep {i} with a mask {shape}")
