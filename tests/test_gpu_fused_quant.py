"""Producers fused with the per-token int8 quantizer (residual add + RMSNorm,
SwiGLU product) against the oracle's unfused chain. The float part carries the
bf16 tolerance; the quantizer part is checked bit-exactly on the kernel's own
bf16 output."""

import pytest
import torch

from oracle import w8a8_oracle as O
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def C():
    from astrai_amd.extension import _cabi
    assert _cabi.load() is not None, _cabi.load_error()
    return _cabi


def _codes_close(got, want, s_got, s_want):
    """codes within one step and >= 98% equal; steps within one bf16 ulp of the row maximum"""
    d = (got.cpu().int() - want.int()).abs()
    assert d.max().item() <= 1, d.max().item()
    assert (d == 0).float().mean().item() >= 0.98
    torch.testing.assert_close(s_got.cpu().reshape(-1), s_want.reshape(-1), rtol=2.0 ** -7, atol=0)


@pytest.mark.parametrize("rows,k,with_res", [(32, 2048, True), (32, 2048, False), (1, 2048, True),
                                             (5, 8, True), (3, 8192, False), (17, 5632, True),
                                             # long blocks without a residual: one wave per row
                                             (2048, 2048, False), (513, 4096, False), (1000, 264, False),
                                             (4099, 512, False), (600, 1024, False), (700, 4104, False),
                                             (2048, 2048, True)])
def test_add_rmsnorm_quantize(C, rows, k, with_res):
    print(f"case rows={rows} k={k} res={with_res}", flush=True)
    g = torch.Generator().manual_seed(rows * 131 + k)
    x = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    res = (torch.randn(rows, k, generator=g) * 0.5).to(torch.bfloat16) if with_res else None
    w = (1.0 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16)
    eps = 1e-5
    xq, s, t, y = C.add_rmsnorm_quantize_int8(x.to(DEV), w.to(DEV), eps, res.to(DEV) if with_res else None,
                                              want_y=True)
    wq, ws, wt, wy = O.add_rmsnorm_quantize_int8(x, w, eps, res)
    if with_res:
        assert torch.equal(t.cpu().view(torch.int16), wt.view(torch.int16))  # one bf16 add: exact
    else:
        assert t is None
    assert_bf16_close(y, wy, what="rmsnorm y")
    # the quantizer on the kernel's own y: bit-exact
    oq, os_ = O.int8_quantize_rows(y.cpu())
    assert torch.equal(xq.cpu(), oq) and torch.equal(s.cpu(), os_)
    _codes_close(xq, wq, s, ws)


@pytest.mark.parametrize("rows,k", [(2048, 2048), (513, 4096), (1000, 264), (600, 1024), (4099, 512), (700, 3080)])
def test_rmsnorm_producer_bits_do_not_depend_on_the_launch_size(C, rows, k):
    """A block of at least 512 rows runs one wave per row, fewer rows one workgroup per row;
    both take the sum of squares in the same order, so a token's y, step and codes are the
    same bits whether it is normalised in a prefill block or in a decode step."""
    print(f"case rows={rows} k={k}", flush=True)
    g = torch.Generator().manual_seed(rows * 7 + k)
    x = (torch.randn(rows, k, generator=g) * torch.exp2(torch.randn(rows, 1, generator=g))).to(torch.bfloat16).to(DEV)
    w = (1.0 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16).to(DEV)
    xq, s, _, y = C.add_rmsnorm_quantize_int8(x, w, 1e-5, None, want_y=True)          # one wave per row
    for lo in range(0, rows, 300):                                                   # one workgroup per row
        pq, ps, _, py = C.add_rmsnorm_quantize_int8(x[lo:lo + 300], w, 1e-5, None, want_y=True)
        assert torch.equal(py.view(torch.int16), y[lo:lo + 300].view(torch.int16)), lo
        assert torch.equal(ps, s[lo:lo + 300]) and torch.equal(pq, xq[lo:lo + 300]), lo


@pytest.mark.parametrize("rows,width,fused_buffer", [(32, 5632, True), (32, 5632, False), (1, 5632, True),
                                                     (7, 8, False), (3, 8192, True)])
def test_silu_mul_quantize(C, rows, width, fused_buffer):
    print(f"case rows={rows} width={width} fused={fused_buffer}", flush=True)
    g = torch.Generator().manual_seed(rows * 17 + width)
    gu = (torch.randn(rows, 2 * width, generator=g) * 2.0).to(torch.bfloat16)
    gate, up = gu[:, :width], gu[:, width:]
    d = gu.to(DEV)
    if fused_buffer:
        hq, s, h = C.silu_mul_quantize_int8(d[:, :width], d[:, width:], want_h=True)
    else:
        hq, s, h = C.silu_mul_quantize_int8(d[:, :width].contiguous(), d[:, width:].contiguous(), want_h=True)
    wq, ws, wh = O.silu_mul_quantize_int8(gate, up)
    assert_bf16_close(h, wh, what="silu*up")
    oq, os_ = O.int8_quantize_rows(h.cpu())
    assert torch.equal(hq.cpu(), oq) and torch.equal(s.cpu(), os_)
    _codes_close(hq, wq, s, ws)


def test_fused_entry_points_reject_unsupported(C):
    x = torch.zeros(2, 12, device=DEV, dtype=torch.bfloat16)   # K % 8 != 0
    w = torch.ones(12, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        C.add_rmsnorm_quantize_int8(x, w, 1e-5)
    big = torch.zeros(1, 8200, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="8192"):
        C.silu_mul_quantize_int8(big, big)


def test_fused_producers_random_shape_sweep(C):
    """Seeded random row counts and widths (multiples of 8 up to 8192) through both producers."""
    g = torch.Generator().manual_seed(808)
    r = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for i in range(12):
        test_add_rmsnorm_quantize(C, r(1, 70), 8 * r(1, 1025), bool(i % 2))
    for i in range(12):
        test_silu_mul_quantize(C, r(1, 70), 8 * r(1, 1025), bool(i % 2))


def _swiglu_case(C, m, width, k, seed):
    """int8 activations and the gate / up weights of one MLP; returns the device tensors and
    what the unblocked chain (GEMM on gate|up, then the producer) gives."""
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8).to(DEV)
    wg = torch.randint(-127, 128, (width, k), generator=g, dtype=torch.int8).to(DEV)
    wu = torch.randint(-127, 128, (width, k), generator=g, dtype=torch.int8).to(DEV)
    # steps sized so that gate covers the range where silu bends (|gate| up to ~8)
    sa = (torch.rand(m, generator=g) * 0.01 + 0.005).to(DEV)
    sg = (torch.rand(width, generator=g) * 0.002 + 0.0005).to(DEV)
    su = (torch.rand(width, generator=g) * 0.002 + 0.0005).to(DEV)
    gu = C.mm_int8(a, torch.cat((wg, wu)), sa, torch.cat((sg, su)))
    want = C.silu_mul_quantize_int8(gu[:, :width], gu[:, width:], want_h=True)
    wgu = C.swiglu_block_rows(wg, wu)
    sgu = C.swiglu_block_rows(sg, su)
    return a, wgu, sa, sgu, gu, want


def test_swiglu_block_rows_layout(C):
    gate = torch.arange(128).reshape(128, 1).repeat(1, 2)
    up = gate + 1000
    b = C.swiglu_block_rows(gate, up)
    assert b.shape == (256, 2)
    assert b[:64, 0].tolist() == list(range(64)) and b[64:128, 0].tolist() == list(range(1000, 1064))
    assert b[128:192, 0].tolist() == list(range(64, 128)) and b[192:, 0].tolist() == list(range(1064, 1128))


@pytest.mark.parametrize("m,width,k", [(4096, 5632, 2048),    # config-4 MLP, 16 x 44 tiles
                                       (3900, 3136, 512),     # ragged rows, last tile half wide (N = 49 * 128)
                                       (8192, 2048, 256)])    # two slabs only
def test_swiglu_gemm_epilogue_bit_equal(C, m, width, k):
    """The gate|up GEMM with the SwiGLU product in its epilogue + the known-maximum quantizer
    against the plain GEMM + producer kernel: h, codes and steps bit for bit; the row maxima
    pieces are the maxima of |h| over 64 columns."""
    print(f"case m={m} width={width} k={k}", flush=True)
    assert C.mm_int8_swiglu_fused_shape(m, 2 * width, k)
    a, wgu, sa, sgu, gu, (wq, ws, wh) = _swiglu_case(C, m, width, k, seed=m + width + k)
    hq, s, h = C.mm_int8_swiglu(a, wgu, sa, sgu, want_h=True)
    assert torch.equal(h.view(torch.int16), wh.view(torch.int16))
    assert torch.equal(s, ws) and torch.equal(hq, wq)
    # against the oracle's chain on the GEMM's own gate|up output (sampled rows: CPU time)
    rows = torch.arange(0, m, max(1, m // 64))
    oq, os_, oh = O.silu_mul_quantize_int8(gu[rows, :width].cpu(), gu[rows, width:].cpu())
    assert_bf16_close(h[rows], oh, what="silu*up")
    _codes_close(hq[rows], oq, s[rows], os_)


@pytest.mark.parametrize("m,width,k", [(1, 5632, 2048), (16, 5632, 2048), (64, 5632, 2048), (200, 320, 256),
                                       (1000, 5632, 2048)])
def test_swiglu_blocked_producer_bit_equal(C, m, width, k):
    """Shapes below the large-tile kernel: plain GEMM on the blocked weight + the producer
    that reads blocked columns equals the unblocked chain bit for bit."""
    print(f"case m={m} width={width} k={k}", flush=True)
    assert not C.mm_int8_swiglu_fused_shape(m, 2 * width, k)
    a, wgu, sa, sgu, gu, (wq, ws, wh) = _swiglu_case(C, m, width, k, seed=7 * m + width + k)
    hq, s, h = C.mm_int8_swiglu(a, wgu, sa, sgu, want_h=True)
    assert torch.equal(h.view(torch.int16), wh.view(torch.int16))
    assert torch.equal(s, ws) and torch.equal(hq, wq)


def test_swiglu_both_routes_agree_and_reject(C):
    a, wgu, sa, sgu, gu, (wq, ws, wh) = _swiglu_case(C, 4096, 3072, 256, seed=99)
    for fused in (True, False):
        hq, s, h = C.mm_int8_swiglu(a, wgu, sa, sgu, want_h=True, fused=fused)
        assert torch.equal(h.view(torch.int16), wh.view(torch.int16)) and torch.equal(hq, wq) and torch.equal(s, ws)
    with pytest.raises(RuntimeError, match="192 output tiles"):
        C.mm_int8_swiglu(a[:64], wgu, sa[:64], sgu, fused=True)
    with pytest.raises(RuntimeError, match="blocks of 64"):
        C.mm_int8_swiglu(a, wgu[:192], sa, sgu[:192])


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("rows,k,with_res", [(32, 2048, True), (5, 8, False), (3, 8192, True), (300, 5632, False)])
def test_add_rmsnorm_quantize_fp8(C, rows, k, with_res, fmt):
    """Per-tensor fp8 twin: value part to the bf16 tolerance against the oracle's chain, the
    codes and the maximum bit-exact against the oracle's fp8 quantizer on the kernel's own y."""
    print(f"case rows={rows} k={k} res={with_res} fmt={fmt}", flush=True)
    g = torch.Generator().manual_seed(rows * 131 + k + fmt)
    x = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    res = (torch.randn(rows, k, generator=g) * 0.5).to(torch.bfloat16) if with_res else None
    w = (1.0 + 0.1 * torch.randn(k, generator=g)).to(torch.bfloat16)
    scale = torch.tensor([3.7 / (57344.0 if fmt else 448.0)])   # some values saturate
    x8, amax, t, y = C.add_rmsnorm_quantize_fp8(x.to(DEV), w.to(DEV), 1e-5, scale.to(DEV),
                                                res.to(DEV) if with_res else None, fmt=fmt, want_y=True)
    _, _, wt, wy = O.add_rmsnorm_quantize_int8(x, w, 1e-5, res)
    if with_res:
        assert torch.equal(t.cpu().view(torch.int16), wt.view(torch.int16))
    assert_bf16_close(y, wy, what="rmsnorm y")
    o8, oamax = O.fp8_quantize_saturating(y.cpu(), scale, fmt)
    assert torch.equal(x8.cpu().view(torch.uint8), o8.view(torch.uint8))
    assert torch.equal(amax.cpu(), oamax)


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("rows,width,fused_buffer", [(32, 5632, True), (7, 8, False), (3, 11008, True)])
def test_silu_mul_quantize_fp8(C, rows, width, fused_buffer, fmt):
    print(f"case rows={rows} width={width} fused={fused_buffer} fmt={fmt}", flush=True)
    g = torch.Generator().manual_seed(rows * 17 + width + fmt)
    gu = (torch.randn(rows, 2 * width, generator=g) * 2.0).to(torch.bfloat16)
    d = gu.to(DEV)
    scale = torch.tensor([6.0 / (57344.0 if fmt else 448.0)])
    gate, up = (d[:, :width], d[:, width:]) if fused_buffer else (d[:, :width].contiguous(), d[:, width:].contiguous())
    prior = torch.tensor([0.25], device=DEV)    # the slot keeps a larger earlier maximum or grows
    h8, amax, h = C.silu_mul_quantize_fp8(gate, up, scale.to(DEV), fmt=fmt, amax=prior, want_h=True)
    _, _, wh = O.silu_mul_quantize_int8(gu[:, :width], gu[:, width:])
    assert_bf16_close(h, wh, what="silu*up")
    o8, oamax = O.fp8_quantize_saturating(h.cpu(), scale, fmt)
    assert torch.equal(h8.cpu().view(torch.uint8), o8.view(torch.uint8))
    assert torch.equal(amax.cpu(), torch.maximum(oamax, torch.tensor([0.25])))
    # same h as the int8 producer forms
    if width <= 8192:
        _, _, hi = C.silu_mul_quantize_int8(gate, up, want_h=True)
        assert torch.equal(h.view(torch.int16), hi.view(torch.int16))


# ---- projections whose output joins the residual stream -----------------------------------------

@pytest.mark.parametrize("m,n,k,bias", [
    (32, 2048, 2048, False),     # config-4 output projection at a decode step (row-range kernel)
    (32, 2048, 5632, False),     # config-4 down projection
    (1, 2048, 2048, False), (1, 2049, 5632, True), (1, 11008, 4096, False), (1, 3, 256, True),   # one token: dot kernel
    (2, 44, 256, True), (17, 3072, 512, True), (64, 2048, 2048, False),
    (100, 1028, 256, False), (128, 2048, 2048, True),
    (48, 11008, 256, True), (64, 8192, 512, False),   # 33..64 tokens on long row ranges
    (16384, 2048, 2048, False),  # config-4 output projection at prefill (large-tile kernel, 64 x 8 tiles)
    (4096, 2048, 5632, False),   # down projection, 16 x 8 tiles = 128 < 192: plain GEMM + addition pass
    (12500, 4096, 256, True),    # large-tile kernel, ragged rows, bias
    (200, 100, 48, True), (3, 7, 16, False), (129, 2050, 256, False),   # shapes without a fused epilogue
])
def test_mm_int8_resid_bit_equal(C, m, n, k, bias):
    """``mm_int8`` + residual in one entry point against the GEMM followed by the bf16 addition
    (what ``attn_output + x`` computes on bf16 tensors): bit for bit, every route; the GEMM
    itself is checked against the oracle on sampled rows."""
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8).to(DEV)
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(DEV)
    sa = (torch.rand(m, generator=g) * 0.01 + 0.005).to(DEV)
    sw = (torch.rand(n, generator=g) * 0.002 + 0.0005).to(DEV)
    b = torch.randn(n, generator=g).bfloat16().to(DEV) if bias else None
    # residual of the product's own magnitude, so that the sum's rounding matters
    r = (torch.randn(m, n, generator=g) * (0.3 * k ** 0.5)).bfloat16().to(DEV)
    y = C.mm_int8(a, w, sa, sw, b)
    want = y + r
    got = C.mm_int8_resid(a, w, sa, sw, r, b)
    assert got.data_ptr() != r.data_ptr()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    rows = torch.arange(0, m, max(1, m // 32))
    oy = O.int8_gemm(a[rows].cpu(), w.cpu(), sa[rows].cpu(), sw.cpu(), None if b is None else b.cpu())
    assert_bf16_close(got[rows], (oy.float() + r[rows].cpu().float()).bfloat16(), what="product + residual")


def test_mm_int8_resid_rejects(C):
    a = torch.zeros(8, 256, dtype=torch.int8, device=DEV)
    w = torch.zeros(16, 256, dtype=torch.int8, device=DEV)
    sa, sw = torch.ones(8, device=DEV), torch.ones(16, device=DEV)
    with pytest.raises(RuntimeError, match="resid"):
        C.mm_int8_resid(a, w, sa, sw, torch.zeros(8, 15, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(RuntimeError, match="resid"):
        C.mm_int8_resid(a, w, sa, sw, torch.zeros(8, 16, dtype=torch.float32, device=DEV))
    # through the C entry point: the output may not overlap the residual
    lib = C.load()
    r = torch.zeros(8, 16, dtype=torch.bfloat16, device=DEV)
    rc = lib.astrai_w8a8_gemm_int8_ptpc_resid(a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), None,
                                              r.data_ptr(), r.data_ptr(), 8, 16, 256, None)
    assert rc != 0 and b"overlaps" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_int8_ptpc_resid(a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), None,
                                              None, r.data_ptr(), 8, 16, 256, None)
    assert rc != 0 and b"residual" in lib.astrai_w8a8_last_error()
    # k == 0: the product is empty, the residual passes through
    r = torch.randn(8, 16, device=DEV).bfloat16()
    out = C.mm_int8_resid(a[:, :0], w[:, :0], sa, sw, r)
    assert torch.equal(out, r)
    # no rows: nothing to launch
    out = C.mm_int8_resid(a[:0], w, sa[:0], sw, r[:0])
    assert out.shape == (0, 16)
