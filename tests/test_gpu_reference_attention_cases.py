"""The reference's own kernel-level attention tests, case for case, against this backend
(tests/extension/test_kernel_mask.py:11-67; the kernel-level part of
tests/extension/test_backend_equivalence.py:166-213). Same shapes (head_dim 64, 4 heads on 1 KV
head; 2 heads on 1 for the decode case), same calls through ``ops``, same assertions, plus the
oracle where the reference only checks the shape. Inputs are drawn on the CPU from a fixed seed."""

import pytest
import torch

from oracle import decoder_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
D = 64  # tests/extension/conftest.py:9


def _qkv(seed, batch=1, q_len=8, n_heads=4, n_kv_heads=1, kv_len=8, d=D):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, q_len, n_heads, d, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, kv_len, n_kv_heads, d, generator=g).to(torch.bfloat16)
    v = torch.randn(batch, kv_len, n_kv_heads, d, generator=g).to(torch.bfloat16)
    return q, k, v


def _check(out, q, k, v, mask):
    want = O.attn_dense(q, k, v, mask=mask)
    err = (out.float().cpu() - want.float()).abs()
    assert (err <= 2e-2 * want.float().abs() + 2.0 ** -6 * want.float().pow(2).mean().sqrt()).all()


def test_kernel_accepts_2d_mask():
    from astrai_amd.extension.ops import attn_prefill
    q, k, v = _qkv(1)
    mask = torch.ones(1, 8, dtype=torch.bool)
    mask[:, 4:] = False
    out = attn_prefill(q.to(DEV), k.to(DEV), v.to(DEV), mask=mask.to(DEV), is_causal=False)
    assert out.shape == (1, 8, 4, D)
    _check(out, q, k, v, mask)


def test_kernel_accepts_3d_mask():
    from astrai_amd.extension.ops import attn_prefill
    q, k, v = _qkv(2)
    mask = torch.ones(1, 8, 8, dtype=torch.bool)
    out = attn_prefill(q.to(DEV), k.to(DEV), v.to(DEV), mask=mask.to(DEV), is_causal=False)
    assert out.shape == (1, 8, 4, D)
    _check(out, q, k, v, mask)


def test_kernel_accepts_4d_mask():
    from astrai_amd.extension.ops import attn_prefill
    q, k, v = _qkv(3)
    mask = torch.ones(1, 1, 8, 8, dtype=torch.bool)
    mask[:, :, :, 4:] = False
    out = attn_prefill(q.to(DEV), k.to(DEV), v.to(DEV), mask=mask.to(DEV), is_causal=False)
    assert out.shape == (1, 8, 4, D)
    _check(out, q, k, v, mask)


@pytest.mark.parametrize("d,q_len,kv_len", [(D, 8, 8), (128, 8, 8), (128, 200, 333)])
def test_4d_mask_matches_no_mask_when_all_true(d, q_len, kv_len):
    """diff == 0.0, as the reference asserts; also at head_dim 128, where the unmasked call runs
    the MFMA kernel's fast path for whole tiles and the masked call its masking path."""
    from astrai_amd.extension.ops import attn_prefill
    q, k, v = (t.to(DEV) for t in _qkv(4, q_len=q_len, kv_len=kv_len, d=d))
    out_no_mask = attn_prefill(q, k, v, mask=None, is_causal=False)
    mask = torch.ones(1, 1, q_len, kv_len, dtype=torch.bool, device=DEV)
    out_with_mask = attn_prefill(q, k, v, mask=mask, is_causal=False)
    diff = (out_no_mask.float() - out_with_mask.float()).abs().max().item()
    assert diff == 0.0, f"4D all-True mask diff: {diff}"
    for causal in (False, True):
        a = attn_prefill(q, k, v, mask=None, is_causal=causal)
        b = attn_prefill(q, k, v, mask=mask, is_causal=causal)
        assert torch.equal(a, b), causal


def test_paged_decode_appends_new_kv_in_kernel():
    """Two requests of 9 and 7 positions in a pool of 8-slot pages; the decode call stores the
    current token's K/V at each request's newest slot, writes into ``out_buf`` and takes the
    split buffers it does not need."""
    from astrai_amd.extension.ops import attn_paged_decode
    g = torch.Generator().manual_seed(5)
    n_tokens, page = 128, 8
    k_buf = torch.randn(n_tokens, 1, D, generator=g).to(torch.bfloat16)
    v_buf = torch.randn(n_tokens, 1, D, generator=g).to(torch.bfloat16)
    lens = [9, 7]
    req_to_token = torch.full((2, 64), -1, dtype=torch.int32)
    pages = [[3, 9], [5]]                      # page numbers of each request, as a page allocator hands them out
    for r, n in enumerate(lens):
        for j in range(n):
            req_to_token[r, j] = pages[r][j // page] * page + j % page
    out_cache_loc = torch.tensor([int(req_to_token[r, lens[r] - 1]) for r in range(2)])
    kv_indptr = torch.tensor([0, 9, 16], dtype=torch.int32)
    q = torch.randn(2, 2, D, generator=g).to(torch.bfloat16)
    new_k = torch.randn(2, 1, D, generator=g).to(torch.bfloat16)
    new_v = torch.randn(2, 1, D, generator=g).to(torch.bfloat16)
    kd, vd = k_buf.to(DEV), v_buf.to(DEV)
    decode_out = torch.zeros(4, 2, D, dtype=torch.bfloat16, device=DEV)
    out = attn_paged_decode(q.to(DEV), kd, vd, req_to_token.to(DEV), torch.arange(2, dtype=torch.int32, device=DEV),
                            kv_indptr.to(DEV), new_k=new_k.to(DEV), new_v=new_v.to(DEV), is_causal=True,
                            o_part_buf=torch.empty(2 * 2 * 16 * D, device=DEV),
                            ml_part_buf=torch.empty(2 * 2 * 16 * 2, device=DEV), out_buf=decode_out)
    torch.cuda.synchronize()
    torch.testing.assert_close(kd[out_cache_loc.to(DEV)].cpu(), new_k, rtol=0, atol=0)
    torch.testing.assert_close(vd[out_cache_loc.to(DEV)].cpu(), new_v, rtol=0, atol=0)
    assert torch.isfinite(out).all()
    assert out.data_ptr() == decode_out.data_ptr()
    kr, vr = k_buf.clone(), v_buf.clone()
    kr[out_cache_loc], vr[out_cache_loc] = new_k, new_v
    want = O.attn_paged_decode(q, kr, vr, req_to_token, torch.arange(2, dtype=torch.int32), kv_indptr)
    assert (out.float().cpu() - want.float()).abs().max().item() < 2e-2


@pytest.mark.parametrize("d,h,hkv", [(D, 2, 1), (128, 16, 4)])
def test_paged_decode_graph_replay_is_exact(d, h, hkv):
    """Kernel-level counterpart of tests/extension/test_backend_equivalence.py:216-272: the decode
    call (new K/V stored, output into ``out_buf``) captured once into a HIP graph and replayed
    while the sequences grow; every replay equals the eager call on the same state, bit for bit.
    Eager work and synchronisations sit between the replays."""
    from astrai_amd.extension.ops import attn_paged_decode
    g = torch.Generator().manual_seed(d + h)
    b, max_ctx, pool = 3, 48, 200
    k_buf = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16).to(DEV)
    v_buf = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16).to(DEV)
    table = torch.randperm(pool, generator=g)[: b * max_ctx].int().reshape(b, max_ctx).to(DEV)
    rows = torch.arange(b, dtype=torch.int32, device=DEV)
    lens = torch.tensor([5, 17, 30])
    q = torch.zeros(b, h, d, dtype=torch.bfloat16, device=DEV)
    new_k = torch.zeros(b, hkv, d, dtype=torch.bfloat16, device=DEV)
    new_v = torch.zeros_like(new_k)
    indptr = torch.zeros(b + 1, dtype=torch.int32, device=DEV)
    out_buf = torch.zeros(b, h, d, dtype=torch.bfloat16, device=DEV)

    def call(kb, vb, out):
        return attn_paged_decode(q, kb, vb, table, rows, indptr, new_k=new_k, new_v=new_v, is_causal=True, out_buf=out)

    def step_inputs(step):
        q.copy_(torch.randn(b, h, d, generator=g).to(torch.bfloat16))
        new_k.copy_(torch.randn(b, hkv, d, generator=g).to(torch.bfloat16))
        new_v.copy_(torch.randn(b, hkv, d, generator=g).to(torch.bfloat16))
        indptr.copy_(torch.tensor([0] + (lens + step).cumsum(0).tolist(), dtype=torch.int32))

    step_inputs(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                     # warm-up off the capture, on copies of the pools
        call(k_buf.clone(), v_buf.clone(), torch.empty_like(out_buf))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(k_buf, v_buf, out_buf)
    for step in range(1, 6):
        step_inputs(step)
        ke, ve = k_buf.clone(), v_buf.clone()          # eager reference on the state before the replay
        want = call(ke, ve, torch.empty_like(out_buf)).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_buf, want), step
        assert torch.equal(k_buf, ke) and torch.equal(v_buf, ve), step
