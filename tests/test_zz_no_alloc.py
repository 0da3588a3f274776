"""The decode-attention entry point that allocates nothing
(``astrai_w8a8_attn_decode_bf16_static_scratch``: the context splits' partial results go
to an array the library holds in static device memory) against the entry point it is
a variant of (``astrai_w8a8_attn_decode_bf16`` with a caller-owned workspace), through
the C ABI: same kernels, so bit-equal outputs; two calls in a row, the second smaller,
share the array."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(b, h, hkv, s, max_len, newest, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, h, s, 128, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, max_len, 128, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.arange(newest - s + 1, newest + 1, dtype=torch.long, device=DEV)
    return q, kc, vc, pos


def _both(lib, q, kc, vc, pos, nsplit):
    """(bf16, int8, steps) of the workspace entry and of the static-scratch entry."""
    from astrai_amd.extension import _cabi
    b, h, s, d = q.shape
    hkv, max_len = kc.size(1), kc.size(2)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.astrai_w8a8_attn_decode_workspace_floats(b, hkv, nsplit, (h // hkv) * s)
    ws = torch.full((need,), float("nan"), device=DEV)
    outs = []
    for static in (False, True):
        out = torch.zeros(b, s, h * d, dtype=torch.bfloat16, device=DEV)
        oq = torch.zeros(b * s, h * d, dtype=torch.int8, device=DEV)
        osc = torch.zeros(b * s, dtype=torch.float32, device=DEV)
        head = (q.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos.data_ptr())
        tail = (out.data_ptr(), oq.data_ptr(), osc.data_ptr(), b, s, h, hkv, d, max_len, nsplit, d ** -0.5, stream)
        if static:
            rc = lib.astrai_w8a8_attn_decode_bf16_static_scratch(*head, *tail)
        else:
            rc = lib.astrai_w8a8_attn_decode_bf16(*head, ws.data_ptr(), ws.numel(), *tail)
        assert rc == 0, lib.astrai_w8a8_last_error()
        outs.append((out, oq, osc))
    torch.cuda.synchronize()
    return outs


def test_static_scratch_entry_equals_workspace_entry_on_two_calls_in_a_row():
    from astrai_amd.extension import _cabi
    lib = _cabi.load()
    assert lib is not None, _cabi.load_error()
    # config-4 decode step (32 sequences, 16 query / 4 KV heads, 3 splits), then a smaller
    # call that reuses the front of the array the first one filled
    for case in ((32, 16, 4, 1, 640, 520, 3), (5, 8, 2, 2, 96, 70, 2)):
        print("case", case, flush=True)
        *shape, nsplit = case
        q, kc, vc, pos = _inputs(*shape, seed=sum(case))
        (w_out, w_q, w_s), (s_out, s_q, s_s) = _both(lib, q, kc, vc, pos, nsplit)
        assert torch.isfinite(w_out.float()).all() and w_out.float().abs().max() > 0
        assert torch.equal(s_out, w_out) and torch.equal(s_q, w_q) and torch.equal(s_s, w_s)
    # the adapter: outputs brought by the caller, nothing allocated
    q, kc, vc, pos = _inputs(4, 16, 4, 1, 64, 40, seed=7)
    want = _cabi.attn_decode(q, kc, vc, pos, nsplit=4)
    got = torch.empty_like(want)
    _cabi.attn_decode_static_scratch(q, kc, vc, pos, out=got, nsplit=4)
    assert torch.equal(got, want)


def test_static_scratch_entry_rejects_what_does_not_fit():
    from astrai_amd.extension import _cabi
    lib = _cabi.load()
    b, hkv, nsplit = 2048, 8, 64       # 2048 * 8 * 64 * 4 rows * 130 floats >> the array
    assert lib.astrai_w8a8_attn_decode_workspace_floats(b, hkv, nsplit, 1) > _cabi.STATIC_SCRATCH_FLOATS
    rc = lib.astrai_w8a8_attn_decode_bf16_static_scratch(16, 16, 16, 16, 16, None, None, b, 1, hkv, hkv, 128,
                                                         64, nsplit, 1.0, None)
    assert rc == 2 and b"scratch" in lib.astrai_w8a8_last_error()


def test_static_scratch_entry_allocates_nothing_and_replays_in_a_graph():
    """What the entry exists for: with the outputs brought by the caller, a call changes
    neither torch's allocator counters nor the free device memory the driver reports, and it
    can be recorded into a HIP graph whose replays (with eager work and synchronisations
    between them, on fresh inputs written into the captured buffers) equal the workspace
    entry's eager result."""
    from astrai_amd.extension import _cabi
    lib = _cabi.load()
    b, h, hkv, s, max_len, newest, nsplit = 8, 16, 4, 1, 256, 200, 4
    q, kc, vc, pos = _inputs(b, h, hkv, s, max_len, newest, seed=11)
    d = 128
    out = torch.zeros(b, s, h * d, dtype=torch.bfloat16, device=DEV)
    oq = torch.zeros(b * s, h * d, dtype=torch.int8, device=DEV)
    osc = torch.zeros(b * s, dtype=torch.float32, device=DEV)

    def call():
        rc = lib.astrai_w8a8_attn_decode_bf16_static_scratch(
            q.data_ptr(), kc.data_ptr(), vc.data_ptr(), pos.data_ptr(), out.data_ptr(), oq.data_ptr(),
            osc.data_ptr(), b, s, h, hkv, d, max_len, nsplit, d ** -0.5, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.astrai_w8a8_last_error()

    call()                      # (the first call on a device looks the array's address up)
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    call()
    torch.cuda.synchronize()
    after = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
    assert after == before, (before, after)
    want = _cabi.attn_decode(q, kc, vc, pos, nsplit=nsplit)
    assert torch.equal(out, want)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call()
    for rep in range(4):
        gen = torch.Generator().manual_seed(100 + rep)
        q.copy_(torch.randn(q.shape, generator=gen).to(torch.bfloat16))
        kc[:, :, : newest + 1].copy_(torch.randn(b, hkv, newest + 1, d, generator=gen).to(torch.bfloat16))
        want = _cabi.attn_decode(q, kc, vc, pos, nsplit=nsplit)      # eager, its own workspace
        wq = torch.empty_like(oq)
        torch.cuda.synchronize()
        out.zero_(); oq.zero_(); osc.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {rep}"
        assert oq.abs().max() > 0 and torch.isfinite(osc).all()
