"""Paged decode attention (token-granular pool + req_to_token + kv_indptr, the
reference's attn_paged_decode interface) against the oracle."""

import pytest
import torch

from oracle import decoder_oracle as D
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _setup(b, h, hkv, lens, max_ctx, pool, seed, n_req=None, holes=False):
    g = torch.Generator().manual_seed(seed)
    d = 128
    n_req = n_req or b + 2
    q = torch.randn(b, h, d, generator=g).to(torch.bfloat16)
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    rows = torch.randperm(n_req, generator=g)[:b].int()
    table = torch.full((n_req, max_ctx), -1, dtype=torch.int32)
    perm = torch.randperm(pool, generator=g)
    nxt = 0
    for i in range(b):
        for j in range(lens[i]):
            table[rows[i], j] = int(perm[nxt]); nxt += 1
        if holes and lens[i] > 3:
            table[rows[i], 1] = -1        # padding inside a sequence: zero key and value
    # slots that no live position maps to hold poison: they must not be read
    unused = perm[nxt:]
    k_pool[unused] = float("nan")
    v_pool[unused] = float("nan")
    indptr = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    return q, k_pool, v_pool, table, rows, indptr


def _run(args, nsplit=0, mask=None, **kw):
    from astrai_amd.extension import _cabi
    dev = [t.to(DEV) for t in args]
    return _cabi.attn_paged_decode(*dev, nsplit=nsplit, mask=None if mask is None else mask.to(DEV), **kw)


@pytest.mark.parametrize("nsplit", [0, 1, 5])
def test_paged_decode_config4_batch_ragged_lengths(nsplit):
    lens = [513, 1, 17, 640, 100, 33, 512, 64] * 4
    args = _setup(32, 16, 4, lens, 640, 32 * 640 + 100, seed=1)
    got = _run(args, nsplit)
    assert got.shape == (32, 16, 128) and got.dtype == torch.bfloat16
    assert_bf16_close(got, D.attn_paged_decode(*args), what=f"paged decode nsplit={nsplit}")


@pytest.mark.parametrize("b,h,hkv,lens,max_ctx", [
    (1, 4, 1, [1], 4),                 # one key
    (3, 8, 8, [16, 15, 17], 40),       # n_rep 1, tile boundaries
    (2, 16, 2, [31, 200], 256),        # n_rep 8
    (4, 4, 2, [0, 5, 0, 9], 16),       # empty sequences give zeros
])
def test_paged_decode_small_shapes(b, h, hkv, lens, max_ctx):
    print(f"case b={b} h={h} hkv={hkv} lens={lens}", flush=True)
    args = _setup(b, h, hkv, lens, max_ctx, sum(lens) + 7, seed=b + h)
    for nsplit in (1, 3):
        assert_bf16_close(_run(args, nsplit), D.attn_paged_decode(*args), what=f"lens={lens} nsplit={nsplit}")


def test_paged_decode_negative_and_out_of_pool_slots_read_as_zeros():
    args = list(_setup(2, 8, 2, [40, 9], 64, 80, seed=3, holes=True))
    want = D.attn_paged_decode(*args)
    assert_bf16_close(_run(args, 2), want, what="holes")
    # a slot number beyond the pool is treated like a negative one, not dereferenced
    table = args[3].clone()
    table[args[4][0].item(), 2] = 10 ** 6
    args2 = list(args); args2[3] = table
    want_table = table.clone(); want_table[table >= 80] = -1
    want2 = D.attn_paged_decode(args[0], args[1], args[2], want_table, args[4], args[5])
    assert_bf16_close(_run(args2, 2), want2, what="slot beyond the pool")


def test_paged_decode_appends_new_kv_like_the_reference_entry():
    """new_k / new_v are persisted at the slot of each sequence's newest position before
    attending (csrc/kernels/attention/layout_policies.cuh:226-252)."""
    from astrai_amd.extension import _cabi
    q, k_pool, v_pool, table, rows, indptr = _setup(3, 8, 2, [12, 1, 30], 32, 64, seed=8)
    g = torch.Generator().manual_seed(80)
    new_k = torch.randn(3, 2, 128, generator=g).to(torch.bfloat16)
    new_v = torch.randn(3, 2, 128, generator=g).to(torch.bfloat16)
    kp, vp = k_pool.clone(), v_pool.clone()
    lens = [12, 1, 30]
    for i in range(3):
        slot = int(table[rows[i], lens[i] - 1])
        kp[slot], vp[slot] = new_k[i], new_v[i]
    want = D.attn_paged_decode(q, kp, vp, table, rows, indptr)
    kd, vd = k_pool.to(DEV), v_pool.to(DEV)
    out_buf = torch.zeros(5, 8, 128, dtype=torch.bfloat16, device=DEV)
    got = _cabi.attn_paged_decode(q.to(DEV), kd, vd, table.to(DEV), rows.to(DEV), indptr.to(DEV),
                                  new_k=new_k.to(DEV), new_v=new_v.to(DEV), out_buf=out_buf)
    assert_bf16_close(got, want, what="append")
    # the caller's split buffer is used as the workspace when it is large enough (and is scribbled on)
    big = torch.full((1 << 20,), float("nan"), device=DEV)
    again = _cabi.attn_paged_decode(q.to(DEV), kd, vd, table.to(DEV), rows.to(DEV), indptr.to(DEV), nsplit=4,
                                    o_part_buf=big, ml_part_buf=torch.empty(8, device=DEV))
    assert_bf16_close(again, want, what="caller's split buffer")
    assert torch.isfinite(big[:64]).any()
    small = _cabi.attn_paged_decode(q.to(DEV), kd, vd, table.to(DEV), rows.to(DEV), indptr.to(DEV), nsplit=4,
                                    o_part_buf=torch.empty(16, device=DEV))
    assert torch.equal(small, again)
    assert got.data_ptr() == out_buf.data_ptr() and torch.equal(out_buf[3:].cpu(), torch.zeros(2, 8, 128, dtype=torch.bfloat16))
    live = torch.isfinite(kp.float()).all(-1).all(-1)
    assert torch.equal(kd.cpu()[live], kp[live]) and torch.equal(vd.cpu()[live], vp[live])


def test_paged_decode_equals_dense_kernel_on_the_same_cache():
    """a pool that is just the dense cache re-indexed: both kernels, same numbers"""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(21)
    b, h, hkv, n = 4, 16, 4, 130
    q = torch.randn(b, h, 128, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, n, 128, generator=g).to(torch.bfloat16).to(DEV)
    dense = _cabi.attn_decode(q.unsqueeze(2).contiguous(), kc, vc, torch.tensor([n - 1], device=DEV), nsplit=4)
    k_pool = kc.permute(0, 2, 1, 3).reshape(b * n, hkv, 128).contiguous()
    v_pool = vc.permute(0, 2, 1, 3).reshape(b * n, hkv, 128).contiguous()
    table = torch.arange(b * n, dtype=torch.int32, device=DEV).reshape(b, n)
    rows = torch.arange(b, dtype=torch.int32, device=DEV)
    indptr = (torch.arange(b + 1, device=DEV) * n).int()
    paged = _cabi.attn_paged_decode(q, k_pool, v_pool, table, rows, indptr, nsplit=4)
    assert torch.equal(paged.reshape(b, -1), dense.reshape(b, -1))


def test_paged_decode_rejects_what_it_does_not_do():
    from astrai_amd.extension import _cabi
    q, k_pool, v_pool, table, rows, indptr = [t.to(DEV) for t in _setup(1, 4, 1, [3], 8, 8, seed=2)]
    ok = torch.ones(1, 8, dtype=torch.bool, device=DEV)
    for bad, msg in ((ok.float(), "bool"), (ok.cpu(), "CUDA"), (ok.expand(2, 8), "batch"), (ok[:, :0], "kv_len")):
        with pytest.raises(RuntimeError, match=msg):
            _cabi.attn_paged_decode(q, k_pool, v_pool, table, rows, indptr, mask=bad)
    with pytest.raises(RuntimeError, match="int32"):
        _cabi.attn_paged_decode(q, k_pool, v_pool, table.long(), rows, indptr)
    with pytest.raises(RuntimeError, match="together"):
        _cabi.attn_paged_decode(q, k_pool, v_pool, table, rows, indptr, new_k=q[:, :1])


@pytest.mark.parametrize("nsplit", [0, 1, 4])
def test_paged_decode_with_a_key_mask(nsplit):
    """The reference's optional mask [batch, positions], True = attend, indexed by sequence
    (not by table row) and position (csrc/kernels/attention/entry_utils.cuh:226-237)."""
    lens = [300, 1, 17, 64, 0, 33]
    args = _setup(6, 16, 4, lens, 320, sum(lens) + 20, seed=12, holes=True)
    g = torch.Generator().manual_seed(5)
    mask = torch.rand(6, 320, generator=g) < 0.6
    mask[3, :64] = False                      # a sequence with every position hidden: zeros
    mask[0, 100:260] = False                  # whole tiles (and whole splits) hidden
    got = _run(args, nsplit, mask=mask)
    assert_bf16_close(got, D.attn_paged_decode(*args, mask=mask), what=f"masked nsplit={nsplit}")
    assert got[3].abs().sum() == 0 and got[4].abs().sum() == 0
    # a mask narrower than the sequences (strided view): the positions past it are hidden
    narrow = torch.ones(6, 640, dtype=torch.bool)[:, 5:205]
    assert narrow.stride(0) == 640
    assert_bf16_close(_run(args, nsplit, mask=narrow), D.attn_paged_decode(*args, mask=narrow), what="narrow mask")
    # an all-True mask is the unmasked kernel, bit for bit
    assert torch.equal(_run(args, nsplit, mask=torch.ones(6, 320, dtype=torch.bool)), _run(args, nsplit))


def test_paged_decode_random_sweep():
    """Twenty-five seeded random batches: sequence lengths from empty to several hundred,
    grouping, split counts, padding slots in every other batch."""
    g = torch.Generator().manual_seed(1618)
    for i in range(25):
        n_rep = (1, 2, 4, 8)[int(torch.randint(0, 4, (1,), generator=g))]
        hkv = int(torch.randint(1, 5, (1,), generator=g))
        b = int(torch.randint(1, 7, (1,), generator=g))
        lens = [int(torch.randint(0, 400, (1,), generator=g)) for _ in range(b)]
        nsplit = (0, 1, 3, 7, 16)[i % 5]
        print(f"case {i}: h={hkv * n_rep}/{hkv} lens={lens} nsplit={nsplit}", flush=True)
        args = _setup(b, hkv * n_rep, hkv, lens, max(lens) + 2, sum(lens) + 9, seed=300 + i, holes=bool(i % 2))
        assert_bf16_close(_run(args, nsplit), D.attn_paged_decode(*args), what=f"sweep {i}")
        if i % 3 == 0:
            mask = torch.rand(b, max(lens) + 2, generator=g) < 0.5
            assert_bf16_close(_run(args, nsplit, mask=mask), D.attn_paged_decode(*args, mask=mask),
                              what=f"sweep {i} with a mask")
