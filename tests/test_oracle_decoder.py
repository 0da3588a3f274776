"""Pins the decoder oracle with what the mathematics fixes, on CPU."""

import torch

from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig, DenseKVCache
from oracle import decoder_oracle as D

CFG = AutoRegressiveLMConfig(vocab_size=97, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                             num_key_value_heads=2, intermediate_size=96, max_position_embeddings=32)


def test_rotary_is_a_rotation_with_relative_position_property():
    torch.manual_seed(0)
    fc = D.rotary_table(16, 32, 10000.0)
    q = torch.randn(1, 32, 1, 16)
    k = torch.randn(1, 32, 1, 16)
    # same vector placed at every position
    q[:] = q[:, :1]
    k[:] = k[:, :1]
    rq, rk = D.apply_rotary(q, fc[None]), D.apply_rotary(k, fc[None])
    torch.testing.assert_close(rq.norm(dim=-1), q.norm(dim=-1), rtol=1e-5, atol=1e-5)  # norm preserved
    torch.testing.assert_close(rq[:, 0], q[:, 0])                                       # position 0 = identity
    # <R_m q, R_n k> depends on m - n only
    d1 = (rq[0, 5, 0] * rk[0, 2, 0]).sum()
    d2 = (rq[0, 20, 0] * rk[0, 17, 0]).sum()
    torch.testing.assert_close(d1, d2, rtol=1e-4, atol=1e-4)
    # adjacent pairs rotate by angle pos * base^(-2i/dim): check pair 0 at position 1 (angle 1 rad)
    x = torch.zeros(1, 2, 1, 16)
    x[0, 1, 0, 0] = 1.0
    y = D.apply_rotary(x, fc[None, :2])
    torch.testing.assert_close(y[0, 1, 0, :2], torch.tensor([torch.cos(torch.tensor(1.0)), torch.sin(torch.tensor(1.0))]))


def test_ntk_rope_scaling_stretches_the_base_by_the_closed_form():
    """rope_scaling {"type": "ntk", "factor": f} multiplies the base by f^(d/(d-2))
    (components/rope.py:27-54): the model's table and the oracle's against angles computed from
    that closed form with Python floats; factor 1, no scaling and a non-NTK type give the plain
    table; the scaled model follows the oracle end to end."""
    import math
    from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig
    from astrai_amd.model.decoder import get_rotary_emb, ntk_base, rotary_base
    d, theta, factor = 64, 10000.0, 4.0
    assert ntk_base(theta, d, factor) == theta * factor ** (d / (d - 2))
    assert rotary_base(None, d, None) == 10000.0 and rotary_base(5e5, d, None) == 5e5
    assert rotary_base(theta, d, {"factor": factor}) == ntk_base(theta, d, factor)          # default type
    assert rotary_base(theta, d, {"type": "linear", "factor": factor}) == theta             # rope.py:47-50
    assert rotary_base(theta, d, {"type": "ntk", "factor": 1.0}) == theta
    table = get_rotary_emb(d, 40, rotary_base(theta, d, {"type": "ntk", "factor": factor}))
    base = theta * factor ** (d / (d - 2))
    for pos, pair in ((0, 0), (1, 0), (7, 3), (39, 31), (23, 17)):
        ang = pos * base ** (-2 * pair / d)
        want = torch.tensor([math.cos(ang), math.sin(ang)])
        # the table rounds the angle to fp32 before cos / sin (reference: freqs.float())
        assert torch.allclose(table[pos, pair], want, atol=2e-6 * max(1.0, ang)), (pos, pair)
    # the highest frequency is stretched least, the lowest by the whole factor^(d/(d-2)) ... ^((d-2)/d) = factor
    plain = get_rotary_emb(d, 40, theta)
    assert torch.equal(table[:, 0], plain[:, 0])                  # pair 0: angle = position, base-free
    ratio = (theta ** (-(d - 2) / d)) / (base ** (-(d - 2) / d))  # slowest pair's wavelength grows by `factor`
    assert abs(ratio - factor) < 1e-9
    cfg = AutoRegressiveLMConfig(vocab_size=97, hidden_size=128, num_hidden_layers=2, num_attention_heads=2,
                                 num_key_value_heads=1, intermediate_size=192, max_position_embeddings=64,
                                 rope_scaling={"type": "ntk", "factor": factor})
    torch.manual_seed(5)
    model = AutoRegressiveLM(cfg).to(torch.bfloat16).eval()
    # (casting the model casts the table, as in the reference, where it is a float buffer too)
    assert torch.equal(model.freqs_cis, get_rotary_emb(64, 64, ntk_base(10000.0, 64, factor)).to(torch.bfloat16))
    assert not torch.equal(model.freqs_cis, get_rotary_emb(64, 64, 10000.0).to(torch.bfloat16))
    ids = torch.randint(0, 97, (2, 24), generator=torch.Generator().manual_seed(6))
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    with torch.no_grad():
        got = model(ids)["logits"]
        want = D.forward(sd, cfg, ids, D.bf16_linear_fn(sd))
        cfg.rope_scaling = None
        unscaled = D.forward(sd, cfg, ids, D.bf16_linear_fn(sd))
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)
    assert not torch.equal(want, unscaled)   # the scaling is not a no-op at 24 positions


def test_repeat_kv_repeats_each_head_in_place():
    x = torch.arange(2 * 3).float().reshape(1, 1, 2, 3)
    y = D.repeat_kv(x, 2)
    assert y.shape == (1, 1, 4, 3)
    assert torch.equal(y[0, 0, 0], y[0, 0, 1]) and torch.equal(y[0, 0, 2], y[0, 0, 3])
    assert torch.equal(y[0, 0, 0], x[0, 0, 0]) and torch.equal(y[0, 0, 2], x[0, 0, 1])


def test_oracle_bf16_path_equals_the_modules_on_cpu():
    """With stock bf16 linears the functional oracle and the nn.Module decoder are the
    same computation written twice (complex vs real rotary, different head plumbing)."""
    torch.manual_seed(1)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, CFG.vocab_size, (2, 9))
    with torch.no_grad():
        want = D.forward(sd, CFG, ids, D.bf16_linear_fn(sd))
        got = model(ids)["logits"]
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)


def test_causality_and_prefill_decode_contract():
    torch.manual_seed(2)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    lin = D.int8_linear_fn(sd)
    ids = torch.randint(0, CFG.vocab_size, (1, 8))
    full = D.forward(sd, CFG, ids, lin)
    # causal: logits at position t do not depend on later tokens
    ids2 = ids.clone()
    ids2[0, 6:] = (ids2[0, 6:] + 1) % CFG.vocab_size
    part = D.forward(sd, CFG, ids2, lin)
    assert torch.equal(full[:, :6], part[:, :6])
    assert not torch.equal(full[:, 6:], part[:, 6:])
    # the module's prefill-then-decode equals its own full forward (dense cache contract,
    # the analogue of tests/module/test_model_forward.py:71-115 in the reference)
    with torch.no_grad():
        whole = model(ids)["logits"]
        cache = DenseKVCache(CFG, 1, 8, "cpu", torch.bfloat16)
        pre = model(ids[:, :5], cache, torch.arange(5))["logits"]
        dec = [model(ids[:, t:t + 1], cache, torch.tensor([t]))["logits"] for t in range(5, 8)]
    torch.testing.assert_close(torch.cat([pre] + dec, 1).float(), whole.float(), atol=2e-2, rtol=2e-2)


def test_oracle_cached_forward_reproduces_the_full_forward():
    """forward_cached (prefill, then one token at a time, then a two-token block) against
    forward with bf16 linears: same arithmetic up to the attention's rounding (SDPA in bf16
    there, float32 softmax here), and the cache ends up holding every position."""
    torch.manual_seed(5)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    hd = CFG.hidden_size // CFG.num_attention_heads
    ids = torch.randint(0, CFG.vocab_size, (2, 11))
    for lin in (D.bf16_linear_fn(sd), D.int8_linear_fn(sd)):
        whole = D.forward(sd, CFG, ids, lin).float()
        kc = torch.zeros(CFG.num_hidden_layers, 2, CFG.num_key_value_heads, 11, hd, dtype=torch.bfloat16)
        vc = torch.zeros_like(kc)
        parts = [D.forward_cached(sd, CFG, ids[:, :6], lin, kc, vc, torch.arange(6))]
        parts += [D.forward_cached(sd, CFG, ids[:, t:t + 1], lin, kc, vc, torch.tensor([t])) for t in range(6, 9)]
        parts += [D.forward_cached(sd, CFG, ids[:, 9:11], lin, kc, vc, torch.arange(9, 11))]
        inc = torch.cat(parts, 1).float()
        scale = whole.abs().max().item()
        assert (inc - whole).abs().max().item() <= 0.03 * scale
        assert torch.nn.functional.cosine_similarity(inc.flatten(), whole.flatten(), dim=0).item() > 0.999
        assert (kc.float().abs().sum(dim=(0, 1, 2, 4)) > 0).all()


def test_int8_path_tracks_bf16_path():
    torch.manual_seed(3)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, CFG.vocab_size, (2, 12))
    a = D.forward(sd, CFG, ids, D.int8_linear_fn(sd)).float().flatten()
    b = D.forward(sd, CFG, ids, D.bf16_linear_fn(sd)).float().flatten()
    assert torch.nn.functional.cosine_similarity(a, b, dim=0).item() > 0.99


def test_attn_cached_closed_forms():
    """Pins the oracle's cached attention: one visible key returns that key's value row;
    equal scores return the mean of the visible value rows; KV heads are shared by
    consecutive query heads."""
    b, h, hkv, s, max_len, d = 2, 4, 2, 2, 6, 8
    g = torch.Generator().manual_seed(0)
    q = torch.randn(b, h, s, d, generator=g)
    kc = torch.randn(b, hkv, max_len, d, generator=g)
    vc = torch.randn(b, hkv, max_len, d, generator=g)
    pos = torch.tensor([0, 3])
    out = D.attn_cached(q, kc, vc, pos).reshape(b, s, h, d)
    for head in range(h):
        torch.testing.assert_close(out[:, 0, head], vc[:, head // 2, 0])          # token 0 sees key 0 only
    kc0 = torch.zeros_like(kc)                                                    # all scores equal
    out0 = D.attn_cached(q, kc0, vc, pos).reshape(b, s, h, d)
    for head in range(h):
        torch.testing.assert_close(out0[:, 1, head], vc[:, head // 2, :4].mean(1))
    # brute force over one (batch, head, token)
    sc = (q[1, 3, 1] @ kc[1, 1, :4].T) / d ** 0.5
    want = torch.softmax(sc, 0) @ vc[1, 1, :4]
    torch.testing.assert_close(out[1, 1, 3], want)


def test_rope_cache_write_is_the_tensor_op_chain():
    """Pins the oracle's rope + cache write: rotation by 90 degrees swaps and negates the pair;
    caches change only at the written positions."""
    b, s, h, hkv, d, max_len = 1, 2, 2, 1, 4, 5
    qkv = torch.arange(b * s * (h + 2 * hkv) * d, dtype=torch.float32).reshape(b, s, -1)
    freqs = torch.zeros(1, s, d // 2, 2)
    freqs[..., 0] = 0.0   # cos
    freqs[..., 1] = 1.0   # sin: rotate every pair by 90 degrees: (e, o) -> (-o, e)
    kc = torch.full((b, hkv, max_len, d), -1.0)
    vc = torch.full((b, hkv, max_len, d), -1.0)
    pos = torch.tensor([1, 4])
    q = D.rope_cache_write(qkv, freqs, pos, kc, vc, h, hkv, d)
    x = qkv[0, 0, :d]
    torch.testing.assert_close(q[0, 0, 0], torch.stack([-x[1], x[0], -x[3], x[2]]))
    kx = qkv[0, 1, h * d:h * d + d]
    torch.testing.assert_close(kc[0, 0, 4], torch.stack([-kx[1], kx[0], -kx[3], kx[2]]))
    torch.testing.assert_close(vc[0, 0, 1], qkv[0, 0, (h + hkv) * d:])
    assert (kc[0, 0, [0, 2, 3]] == -1).all() and (vc[0, 0, [0, 2, 3]] == -1).all()


def test_paged_decode_oracle_equals_dense_attention_on_a_scattered_cache():
    """Scatter a dense cache into a pool through a random slot table: the paged oracle must
    reproduce the dense one (attn_cached) for every sequence length, including the unused
    tail of each request row and rows of other requests in between."""
    g = torch.Generator().manual_seed(12)
    b, h, hkv, d, max_ctx = 3, 8, 2, 16, 20
    lens = [20, 7, 1]
    pool = 97
    q = torch.randn(b, h, d, generator=g).to(torch.bfloat16)
    dense_k = torch.randn(b, hkv, max_ctx, d, generator=g).to(torch.bfloat16)
    dense_v = torch.randn(b, hkv, max_ctx, d, generator=g).to(torch.bfloat16)
    perm = torch.randperm(pool, generator=g)
    rows = torch.tensor([4, 0, 2])                       # request rows in a table of 5
    table = torch.full((5, max_ctx), -1, dtype=torch.int32)
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)   # other tenants' data
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    nxt = 0
    for i in range(b):
        for j in range(lens[i]):
            slot = int(perm[nxt]); nxt += 1
            table[rows[i], j] = slot
            k_pool[slot] = dense_k[i, :, j]
            v_pool[slot] = dense_v[i, :, j]
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    got = D.attn_paged_decode(q, k_pool, v_pool, table, rows.int(), indptr)
    for i in range(b):
        want = D.attn_cached(q[i:i + 1].unsqueeze(2), dense_k[i:i + 1], dense_v[i:i + 1],
                             torch.tensor([lens[i] - 1]))
        assert torch.equal(got[i].reshape(-1), want.reshape(-1)), i


def test_paged_decode_oracle_single_key_and_empty_sequence():
    """one visible key: the output is that key's value row; no key: zeros"""
    q = torch.randn(2, 4, 8).to(torch.bfloat16)
    k_pool = torch.randn(6, 2, 8).to(torch.bfloat16)
    v_pool = torch.randn(6, 2, 8).to(torch.bfloat16)
    table = torch.tensor([[5, -1, -1], [3, 1, 2]], dtype=torch.int32)
    out = D.attn_paged_decode(q, k_pool, v_pool, table, torch.tensor([0, 1], dtype=torch.int32),
                              torch.tensor([0, 1, 1], dtype=torch.int32))
    assert torch.equal(out[0], v_pool[5].repeat_interleave(2, dim=0))
    assert torch.equal(out[1], torch.zeros(4, 8, dtype=torch.bfloat16))


def test_paged_prefill_oracle_equals_dense_attention_per_sequence():
    """Ragged sequences scattered into a pool: for each one the paged-prefill oracle must equal
    the dense oracle (attn_cached) fed with that sequence alone and positions
    kv_len - q_len + i -- chunked prefill (cached context first) and whole-prompt prefill."""
    g = torch.Generator().manual_seed(31)
    h, hkv, d, max_ctx, pool = 4, 2, 16, 24, 80
    kv_lens, q_lens = [24, 9, 5], [7, 9, 1]
    dense_k = torch.randn(3, hkv, max_ctx, d, generator=g).to(torch.bfloat16)
    dense_v = torch.randn(3, hkv, max_ctx, d, generator=g).to(torch.bfloat16)
    perm = torch.randperm(pool, generator=g)
    rows = torch.tensor([2, 0, 3], dtype=torch.int32)
    table = torch.full((4, max_ctx), -1, dtype=torch.int32)
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    nxt = 0
    for i in range(3):
        for j in range(kv_lens[i]):
            slot = int(perm[nxt]); nxt += 1
            table[rows[i], j] = slot
            k_pool[slot], v_pool[slot] = dense_k[i, :, j], dense_v[i, :, j]
    qo = torch.tensor([0, 7, 16, 17], dtype=torch.int32)
    kvp = torch.tensor([0, 24, 33, 38], dtype=torch.int32)
    q = torch.randn(17, h, d, generator=g).to(torch.bfloat16)
    got = D.attn_paged_prefill(q, k_pool, v_pool, table, rows, kvp, qo, causal=True)
    for i in range(3):
        qi = q[qo[i]:qo[i + 1]].permute(1, 0, 2).unsqueeze(0)                  # [1, H, q_len, D]
        pos = kv_lens[i] - q_lens[i] + torch.arange(q_lens[i])
        want = D.attn_cached(qi, dense_k[i:i + 1], dense_v[i:i + 1], pos)      # [1, q_len, H*D]
        assert torch.equal(got[qo[i]:qo[i + 1]].reshape(q_lens[i], -1), want[0]), i
    # without the causal flag every row sees all kv_len keys
    full = D.attn_paged_prefill(q, k_pool, v_pool, table, rows, kvp, qo, causal=False)
    qi = q[0:7].permute(1, 0, 2).unsqueeze(0)
    want = D.attn_cached(qi, dense_k[0:1], dense_v[0:1], torch.full((7,), 23))
    assert torch.equal(full[0:7].reshape(7, -1), want[0])


def test_paged_oracles_read_a_negative_slot_as_a_zero_key_and_value():
    """The reference gates the K/V load on the slot and the mask on the position only
    (csrc/kernels/attention/layout_policies.cuh:104-110,212-219; prefill_split_q_mma.cuh:84-89,
    121-124; decode_split_kv_mma.cuh:75-82,107-110): a negative table entry inside a sequence
    must act exactly like a slot whose key and value rows are zero -- still attended, score 0 --
    and not like a shorter sequence."""
    g = torch.Generator().manual_seed(21)
    h, hkv, d, pool = 4, 2, 16, 40
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    k_pool[pool - 1] = 0          # a real slot holding a zero key and a zero value
    v_pool[pool - 1] = 0
    lens = [9, 5]
    rows = torch.tensor([1, 0], dtype=torch.int32)
    table = torch.full((2, 12), -1, dtype=torch.int32)
    table[1, :9] = torch.arange(9, dtype=torch.int32)
    table[0, :5] = torch.arange(20, 25, dtype=torch.int32)
    holes = table.clone(); holes[1, 3] = -1; holes[0, 0] = -1
    zeros = table.clone(); zeros[1, 3] = pool - 1; zeros[0, 0] = pool - 1
    indptr = torch.tensor([0, 9, 14], dtype=torch.int32)
    q1 = torch.randn(2, h, d, generator=g).to(torch.bfloat16)
    a = D.attn_paged_decode(q1, k_pool, v_pool, holes, rows, indptr)
    b = D.attn_paged_decode(q1, k_pool, v_pool, zeros, rows, indptr)
    assert torch.equal(a, b)
    short = D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr)
    assert not torch.equal(a, short)
    qo = torch.tensor([0, 9, 12], dtype=torch.int32)      # whole prompt; a 3-row chunk after 2 cached
    qp = torch.randn(12, h, d, generator=g).to(torch.bfloat16)
    for causal in (True, False):
        a = D.attn_paged_prefill(qp, k_pool, v_pool, holes, rows, indptr, qo, causal=causal)
        b = D.attn_paged_prefill(qp, k_pool, v_pool, zeros, rows, indptr, qo, causal=causal)
        assert torch.equal(a, b), causal
    # row 0 of the second sequence sees positions 0..2, all real except the hole at 0
    assert a.abs().sum() > 0


def test_paged_oracles_mask_hides_positions_like_removing_them():
    """The reference's optional mask (csrc/kernels/attention/entry_utils.cuh:226-237,326-346;
    mma_utils.cuh:190-199) is indexed by sequence (not by the row of req_to_token), query row
    inside the sequence and position, True = attend, and is combined with the causal range by
    "and". Pinned by what softmax attention fixes: hiding a position equals a sequence that
    never held it; an all-True mask changes nothing; the lower triangle as a mask equals the
    causal flag; a 2D mask equals its 4D broadcast; hiding everything gives zeros."""
    g = torch.Generator().manual_seed(33)
    h, hkv, d, pool = 4, 2, 16, 64
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    lens = [9, 6]
    rows = torch.tensor([2, 0], dtype=torch.int32)          # sequence 0 lives in table row 2
    table = torch.full((3, 12), -1, dtype=torch.int32)
    table[2, :9] = torch.arange(30, 39, dtype=torch.int32)
    table[0, :6] = torch.arange(10, 16, dtype=torch.int32)
    indptr = torch.tensor([0, 9, 15], dtype=torch.int32)
    q1 = torch.randn(2, h, d, generator=g).to(torch.bfloat16)
    plain = D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr)
    assert torch.equal(D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr,
                                           mask=torch.ones(2, 12, dtype=torch.bool)), plain)
    # hide positions 2 and 7 of sequence 0 and position 0 of sequence 1
    mask = torch.ones(2, 12, dtype=torch.bool)
    mask[0, 2] = mask[0, 7] = mask[1, 0] = False
    got = D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr, mask=mask)
    cut = torch.full((3, 12), -1, dtype=torch.int32)
    cut[2, :7] = torch.tensor([30, 31, 33, 34, 35, 36, 38], dtype=torch.int32)
    cut[0, :5] = torch.arange(11, 16, dtype=torch.int32)
    want = D.attn_paged_decode(q1, k_pool, v_pool, cut, rows, torch.tensor([0, 7, 12], dtype=torch.int32))
    assert (got.float() - want.float()).abs().max() < 2e-2 and not torch.equal(got, plain)
    # a mask narrower than a sequence hides the rest; hiding everything gives zeros
    narrow = D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr, mask=torch.ones(2, 4, dtype=torch.bool))
    first4 = D.attn_paged_decode(q1, k_pool, v_pool, table, rows, torch.tensor([0, 4, 8], dtype=torch.int32))
    assert torch.equal(narrow, first4)
    none = mask.clone(); none[1] = False
    assert D.attn_paged_decode(q1, k_pool, v_pool, table, rows, indptr, mask=none)[1].abs().sum() == 0

    # prefill: whole prompts (q_len == kv_len)
    qo = torch.tensor([0, 9, 15], dtype=torch.int32)
    qp = torch.randn(15, h, d, generator=g).to(torch.bfloat16)
    causal = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True)
    tri = torch.tril(torch.ones(9, 12, dtype=torch.bool))[None, None].expand(2, 1, 9, 12)
    as_mask = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=False, mask=tri)
    assert torch.equal(as_mask, causal)
    both = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True, mask=tri)
    assert torch.equal(both, causal)
    m2 = mask
    m4 = mask[:, None, None, :]
    a = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True, mask=m2)
    b = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True, mask=m4)
    c = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True,
                             mask=m4.expand(2, h, 9, 12))
    assert torch.equal(a, b) and torch.equal(a, c) and not torch.equal(a, causal)
    # row 0 of sequence 1 sees only position 0, which the mask hides: zeros
    assert a[9].abs().sum() == 0 and a[10].abs().sum() > 0
    # a per-head mask: head 1 of sequence 0 loses position 0, the other heads keep it
    per_head = torch.ones(2, h, 9, 12, dtype=torch.bool)
    per_head[0, 1, :, 0] = False
    e = D.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, causal=True, mask=per_head)
    assert torch.equal(e[:, [0, 2, 3]], causal[:, [0, 2, 3]]) and torch.equal(e[9:], causal[9:])
    assert e[0, 1].abs().sum() == 0 and not torch.equal(e[1:9, 1], causal[1:9, 1])


def test_attn_dense_oracle_against_sdpa_and_the_paged_oracle():
    """The dense-entry oracle, pinned on the CPU by a library routine (torch's scaled-dot-product
    attention in float32: causal flag, boolean mask, grouped heads expanded by hand) and by the
    paged oracle on the same keys addressed through an identity table."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(8)
    b, h, hkv, lq, lk, d = 2, 4, 2, 5, 9, 16
    q = torch.randn(b, lq, h, d, generator=g)
    k = torch.randn(b, lk, hkv, d, generator=g)
    v = torch.randn(b, lk, hkv, d, generator=g)
    kx, vx = k.repeat_interleave(2, dim=2), v.repeat_interleave(2, dim=2)
    sd = lambda **kw: F.scaled_dot_product_attention(q.transpose(1, 2), kx.transpose(1, 2), vx.transpose(1, 2), **kw).transpose(1, 2)
    assert torch.allclose(D.attn_dense(q, k, v), sd(), atol=1e-5)
    # bottom-right aligned causal range = offset kv_len - q_len
    band = torch.arange(lk)[None, :] <= torch.arange(lq)[:, None] + (lk - lq)
    assert torch.allclose(D.attn_dense(q, k, v, causal_offset=lk - lq), sd(attn_mask=band), atol=1e-5)
    # top-left aligned (offset 0) is SDPA's is_causal
    assert torch.allclose(D.attn_dense(q, k, v, causal_offset=0), sd(is_causal=True), atol=1e-5)
    m3 = torch.rand(b, lq, lk, generator=g) < 0.7
    m3[..., 0] = True
    assert torch.allclose(D.attn_dense(q, k, v, mask=m3), sd(attn_mask=m3[:, None]), atol=1e-5)
    m2 = m3[:, 0]
    assert torch.allclose(D.attn_dense(q, k, v, mask=m2, causal_offset=lk - lq),
                          sd(attn_mask=m2[:, None, None, :] & band), atol=1e-5)
    # layout 0 is the same numbers transposed
    a0 = D.attn_dense(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), mask=m3, layout=0)
    assert torch.equal(a0.transpose(1, 2), D.attn_dense(q, k, v, mask=m3))
    # the paged oracle over an identity table
    table = torch.arange(b * lk, dtype=torch.int32).reshape(b, lk)
    rows = torch.arange(b, dtype=torch.int32)
    kvp = (torch.arange(b + 1) * lk).int()
    qo = (torch.arange(b + 1) * lq).int()
    paged = D.attn_paged_prefill(q.reshape(b * lq, h, d), k.reshape(b * lk, hkv, d), v.reshape(b * lk, hkv, d),
                                 table, rows, kvp, qo, causal=True, mask=m3[:, None])
    assert torch.allclose(paged.reshape(b, lq, h, d), D.attn_dense(q, k, v, mask=m3, causal_offset=lk - lq), atol=1e-6)
    # a hidden row gives zeros, not NaN
    none = m3.clone(); none[1, 2] = False
    assert D.attn_dense(q, k, v, mask=none)[1, 2].abs().sum() == 0
