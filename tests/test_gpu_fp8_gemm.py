"""fp8 kernels vs the oracle with the reference's own shapes and tolerances
(tests/extension/test_fp8_mma.py:42-198), plus 128-block scaling."""

import pytest
import torch

from oracle import w8a8_oracle as O
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from astrai_amd.extension import get_module, is_available
    from astrai_amd.extension.ops import fp8
    assert is_available("fp8_mm")
    return fp8


def _scale(t):
    return (t.abs().amax().float() / 448.0).clamp_min(1e-12).reshape(1)


@pytest.mark.parametrize("m,n,k", [(16, 8, 32), (17, 9, 33), (31, 15, 64), (32, 48, 96)])
def test_fused_fp8_mm_matches_explicit_quantization(ops, m, n, k):
    # test_fp8_mma.py:42-61 (same seeds, same tolerance), expectation from the oracle
    from astrai_amd.extension import get_module
    print(f"case m={m} n={n} k={k}", flush=True)
    torch.manual_seed(m + n + k)
    a = torch.randn(m, k).to(torch.bfloat16)
    b = torch.randn(n, k).to(torch.bfloat16)
    sa, sb = _scale(a), _scale(b)
    out = get_module("fp8_mm").fp8_mm(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV))
    a8, _ = O.fp8_quantize(a, sa, 0)
    b8, _ = O.fp8_quantize(b, sb, 0)
    expected = O.fp8_gemm(a8, b8, sa, sb)
    assert out.dtype == torch.bfloat16 and out.shape == (m, n)
    torch.testing.assert_close(out.cpu(), expected, atol=0.125, rtol=0.01)
    assert_bf16_close(out, expected, what="fp8_mm")


def test_linear_forward_with_bias_and_amax(ops):
    # test_fp8_mma.py:88-116 forward half: seed 7, 19x13x37, bias, amax equalities
    torch.manual_seed(7)
    m, n, k = 19, 13, 37
    x = torch.randn(m, k).to(torch.bfloat16)
    w = torch.randn(n, k).to(torch.bfloat16)
    _ = torch.randn(m, n)
    bias = torch.randn(n).to(torch.bfloat16)
    sx, sw = _scale(x), _scale(w)
    out, ax, aw = ops.linear_forward_fp8(x.to(DEV), w.to(DEV), bias.to(DEV), sx.to(DEV), sw.to(DEV))
    want, wax, waw = O.linear_forward_fp8(x, w, bias, sx, sw)
    torch.testing.assert_close(out.cpu(), want, atol=0.125, rtol=0.01)
    assert_bf16_close(out, want, what="linear_forward_fp8")
    assert ax.item() == wax.item() and aw.item() == waw.item()
    out3, _, _ = ops.linear_forward_fp8(x.reshape(1, m, k).to(DEV), w.to(DEV), None, sx.to(DEV), sw.to(DEV))
    assert out3.shape == (1, m, n)


def test_linear_backward_fp8_both_formats(ops):
    # test_fp8_mma.py:88-145 backward halves
    for seed, (m, n, k), fmt, gmul, tol in [(7, (19, 13, 37), "e4m3", 1.0, (0.125, 0.01)),
                                            (5, (32, 16, 64), "e5m2", 10.0, (0.5, 0.05))]:
        torch.manual_seed(seed)
        x = torch.randn(m, k).to(torch.bfloat16)
        w = torch.randn(n, k).to(torch.bfloat16)
        g = (torch.randn(m, n) * gmul).to(torch.bfloat16)
        sx, sw, sg = _scale(x), _scale(w), _scale(g)
        if fmt == "e5m2":
            sx, sw, sg = sx * 448 / 57344, sw * 448 / 57344, sg * 448 / 57344
        gx, gw, gb, amax_g = ops.linear_backward_fp8(
            g.to(DEV), x.to(DEV), w.to(DEV), [1, 1, 1], sg.to(DEV), sw.to(DEV), sx.to(DEV), fmt)
        f = 1 if fmt == "e5m2" else 0
        qg = O.fp8_quantize(g, sg, f)[0].float()
        qw = O.fp8_quantize(w, sw, f)[0].float()
        qx = O.fp8_quantize(x, sx, f)[0].float()
        torch.testing.assert_close(gx.cpu(), (qg @ qw * sg * sw).to(torch.bfloat16), atol=tol[0], rtol=tol[1])
        torch.testing.assert_close(gw.cpu(), (qg.t() @ qx * sg * sx).to(torch.bfloat16), atol=tol[0], rtol=tol[1])
        torch.testing.assert_close(gb.cpu(), g.sum(0).to(torch.bfloat16))
        assert amax_g.item() == g.abs().max().item()


@pytest.mark.parametrize("masks", [[1, 0, 0], [0, 1, 0], [0, 0, 1], [0, 0, 0], [1, 1, 0]])
def test_linear_backward_fp8_masks(ops, masks):
    """Each output-mask combination of mm.cu:293-319: unrequested gradients are not
    computed, and amax_g is measured on the dX branch (or when neither GEMM runs) only."""
    print(f"case masks={masks}", flush=True)
    torch.manual_seed(21)
    m, n, k = 69, 24, 40  # 3 x 23 tokens
    x = torch.randn(3, 23, k).to(torch.bfloat16)
    w = torch.randn(n, k).to(torch.bfloat16)
    g = torch.randn(3, 23, n).to(torch.bfloat16)
    sx, sw, sg = _scale(x), _scale(w), _scale(g)
    gx, gw, gb, amax_g = ops.linear_backward_fp8(
        g.to(DEV), x.to(DEV), w.to(DEV), masks, sg.to(DEV), sw.to(DEV), sx.to(DEV), "e4m3")
    qg = O.fp8_quantize(g.reshape(m, n), sg, 0)[0].float()
    qw = O.fp8_quantize(w, sw, 0)[0].float()
    qx = O.fp8_quantize(x.reshape(m, k), sx, 0)[0].float()
    assert gx.shape == x.shape and gw.shape == w.shape
    if masks[0]:
        torch.testing.assert_close(gx.cpu().reshape(m, k), (qg @ qw * sg * sw).to(torch.bfloat16),
                                   atol=0.125, rtol=0.01)
    if masks[1]:
        torch.testing.assert_close(gw.cpu(), (qg.t() @ qx * sg * sx).to(torch.bfloat16),
                                   atol=0.125, rtol=0.01)
    if masks[2]:
        torch.testing.assert_close(gb.cpu(), g.reshape(m, n).sum(0).to(torch.bfloat16))
    else:
        assert gb.numel() == 0
    want_amax = g.abs().max().item() if (masks[0] or not masks[1]) else 0.0
    assert amax_g.item() == want_amax


def test_linear_backward_fp8_4096(ops):
    """Full-size backward (4096 tokens, 4096 x 4096 weight): both GEMMs against
    fp64 products of the oracle's codes, the tolerance of test_fp8_mma.py:149-174."""
    torch.manual_seed(13)
    m = n = k = 4096
    x = torch.randn(m, k).to(torch.bfloat16)
    w = torch.randn(n, k).to(torch.bfloat16)
    g = torch.randn(m, n).to(torch.bfloat16)
    sx, sw, sg = _scale(x), _scale(w), _scale(g)
    gx, gw, gb, amax_g = ops.linear_backward_fp8(
        g.to(DEV), x.to(DEV), w.to(DEV), [1, 1, 1], sg.to(DEV), sw.to(DEV), sx.to(DEV), "e4m3")
    qg = O.fp8_quantize(g, sg, 0)[0].float()
    qw = O.fp8_quantize(w, sw, 0)[0].float()
    qx = O.fp8_quantize(x, sx, 0)[0].float()
    assert_bf16_close(gx, (qg @ qw * sg * sw).to(torch.bfloat16), what="dX 4096")
    assert_bf16_close(gw, (qg.t() @ qx * sg * sx).to(torch.bfloat16), what="dW 4096")
    assert amax_g.item() == g.abs().max().item()


def test_mm_fp8_k4096_vs_float64_and_oracle(ops):
    # test_fp8_mma.py:149-174: seed 11, 512x4096x4096, sa 2.5, sb 1.5, atol 6 / rtol .05 vs fp64
    torch.manual_seed(11)
    m, n, k = 512, 4096, 4096
    a = torch.randn(m, k).to(torch.bfloat16)
    b = torch.randn(n, k).to(torch.bfloat16)
    sa, sb = torch.tensor([2.5]), torch.tensor([1.5])
    a8, _ = ops.quantize_bf16(a.to(DEV), sa.to(DEV), "e4m3")
    b8, _ = ops.quantize_bf16(b.to(DEV), sb.to(DEV), "e4m3")
    out = ops.mm_fp8(a8, b8, sa.to(DEV), sb.to(DEV))
    assert out.dtype == torch.bfloat16 and out.shape == (m, n)
    ra8, _ = O.fp8_quantize(a, sa, 0)
    rb8, _ = O.fp8_quantize(b, sb, 0)
    assert torch.equal(a8.cpu().view(torch.uint8), ra8.view(torch.uint8))
    ref64 = (ra8.double() @ rb8.double().t() * 2.5 * 1.5).to(torch.bfloat16)
    torch.testing.assert_close(out.cpu(), ref64, atol=6.0, rtol=0.05)
    assert_bf16_close(out, O.fp8_gemm(ra8, rb8, sa, sb), what="mm_fp8 k4096")


def test_mm_fp8_fp8_output(ops):
    # test_fp8_mma.py:177-198: seed 12, 256x128x64, scales 2 / 1 / .5
    torch.manual_seed(12)
    m, n, k = 256, 128, 64
    a = torch.randn(m, k).to(torch.bfloat16)
    b = torch.randn(n, k).to(torch.bfloat16)
    sa, sb, os_ = torch.tensor([2.0]), torch.tensor([1.0]), torch.tensor([0.5])
    a8, _ = O.fp8_quantize(a, sa, 0)
    b8, _ = O.fp8_quantize(b, sb, 0)
    out8 = ops.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV), out_dtype="e4m3", out_scale=os_.to(DEV))
    assert out8.dtype == torch.float8_e4m3fn and out8.shape == (m, n)
    want = O.fp8_gemm(a8, b8, sa, sb, 1, os_)
    ref64 = (a8.double() @ b8.double().t() * 2.0 * 1.0 * 0.5).to(torch.bfloat16)
    torch.testing.assert_close(out8.float().cpu().to(torch.bfloat16), ref64, atol=6.0, rtol=0.05)
    # codes agree with the oracle except where the fp32 sum sits on an e4m3 rounding
    # boundary (the MFMA's summation order differs from sgemm's): never more than one
    # code step apart, and rarely
    got_c, want_c = out8.cpu().view(torch.uint8).int(), want.view(torch.uint8).int()
    diff = (got_c - want_c).abs()
    assert diff.max().item() <= 1
    assert (diff != 0).float().mean().item() < 0.01


def test_reference_hand_vectors_on_device(ops, golden):
    kat = golden("reference_kats.json")
    k1, k2 = kat["mm_fp8_cpu"], kat["mm_fp8_fp8_out_cpu"]
    a8 = torch.tensor(k1["a8"]).to(torch.float8_e4m3fn).to(DEV)
    b8 = torch.tensor(k1["b8"]).to(torch.float8_e4m3fn).to(DEV)
    sa, sb = torch.tensor([k1["sa"]], device=DEV), torch.tensor([k1["sb"]], device=DEV)
    assert ops.mm_fp8(a8, b8, sa, sb).cpu().tolist() == k1["out_bf16"]
    os_ = torch.tensor([k2["out_scale"]], device=DEV)
    assert ops.mm_fp8(a8, b8, sa, sb, "e4m3", os_).float().cpu().tolist() == k2["out_e4m3"]


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("m,n,k", [(64, 64, 128), (129, 257, 272), (256, 256, 512), (300, 500, 1040)])
def test_mm_fp8_both_formats_tile_edges(ops, fmt, m, n, k):
    print(f"case fmt={fmt} m={m} n={n} k={k}", flush=True)
    a, b, _ = O.make_inputs(1, m, n, k, w_std=1.0)
    name = "e5m2" if fmt else "e4m3"
    sa, sb = O.dynamic_scale(a, name).reshape(1), O.dynamic_scale(b, name).reshape(1)
    a8, _ = O.fp8_quantize(a, sa, fmt)
    b8, _ = O.fp8_quantize(b, sb, fmt)
    out = ops.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm(a8, b8, sa, sb), what=f"mm_fp8 {name}")


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("m,n,k", [(300, 520, 1032), (64, 1024, 1288), (513, 257, 2047)])
def test_mm_fp8_k_not_in_16_byte_pieces_zero_padded(ops, fmt, m, n, k):
    """K % 16 != 0 on a product large enough for the wrapper to zero-pad the rows for the tuned
    kernels: zero codes add nothing, the result stays within the GEMM's tolerance of the oracle."""
    from astrai_amd.extension import _cabi
    print(f"case fmt={fmt} m={m} n={n} k={k}", flush=True)
    assert k % 16 and m * n * k >= _cabi._PAD_K_MIN_MACS
    a, b, _ = O.make_inputs(1, m, n, k, w_std=1.0)
    name = "e5m2" if fmt else "e4m3"
    sa, sb = O.dynamic_scale(a, name).reshape(1), O.dynamic_scale(b, name).reshape(1)
    a8, _ = O.fp8_quantize(a, sa, fmt)
    b8, _ = O.fp8_quantize(b, sb, fmt)
    ad, bd = a8.to(DEV), b8.to(DEV)
    pa, pb, kp = _cabi._pad_k(ad, bd)
    assert kp % 128 == 0 and pa.dtype == ad.dtype and pa.shape == (m, kp) and pb.shape == (n, kp)
    assert torch.equal(pa[:, :k].view(torch.uint8), ad.view(torch.uint8)) and not pa[:, k:].view(torch.uint8).any()
    out = ops.mm_fp8(ad, bd, sa.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm(a8, b8, sa, sb), what=f"mm_fp8 {name} padded K")
    sa_r = (torch.rand(m, 1, generator=torch.Generator().manual_seed(k)) * 0.5 + 0.5) * sa
    out = ops.mm_fp8(ad, bd, sa_r.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm(a8, b8, sa_r, sb), what=f"mm_fp8 {name} padded K, row scales")


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("m,n,k", [(1, 11008, 4096), (4, 11008, 4096), (16, 3072, 2048), (33, 2048, 5632),
                                   (64, 11008, 4096), (7, 1001, 512), (48, 130, 256), (17, 6144, 2048),
                                   (65, 3072, 2048), (96, 11008, 4096), (128, 2048, 5632), (113, 777, 768)])
def test_mm_fp8_decode_shapes_row_range_kernel(ops, fmt, m, n, k):
    """At most 128 activation rows with K % 256 == 0: the row-range decode kernel on fp8 operands
    (weights streamed once, fp32 partials of the waves added in a fixed order). Per-tensor steps
    with and without bias, one step per row and column, and the raw fp32 accumulator."""
    from astrai_amd.extension import _cabi
    print(f"case fmt={fmt} m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(11 * m + 5 * n + k + fmt)
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    a8 = (torch.randn(m, k, generator=g) * 1.5).to(dt)
    b8 = (torch.randn(n, k, generator=g) * 1.5).to(dt)
    sa, sb = torch.tensor([0.37]), torch.tensor([0.011])
    ad, bd = a8.to(DEV), b8.to(DEV)
    out = ops.mm_fp8(ad, bd, sa.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm(a8, b8, sa, sb), what="decode rows, per tensor")
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    out = _cabi.mm_fp8(ad, bd, sa.to(DEV), sb.to(DEV), 0, None, bias.to(DEV))
    assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa, sb, bias), what="decode rows, bias")
    sa_r = torch.exp2(torch.rand(m, 1, generator=g) * 6.0 - 3.0)
    sb_r = torch.exp2(torch.rand(n, generator=g) * 6.0 - 3.0)
    out = _cabi.mm_fp8(ad, bd, sa_r.to(DEV), sb_r.to(DEV), 0, None, bias.to(DEV))
    assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa_r, sb_r, bias), what="decode rows, row/column steps")
    acc = _cabi.mm_fp8_acc(ad, bd).cpu()
    want = a8.double() @ b8.double().t()
    bound = (a8.double().abs() @ b8.double().abs().t()) * 2.0 ** -16 + 1e-30
    assert acc.dtype == torch.float32 and bool(((acc.double() - want).abs() <= bound).all())
    # the same call twice gives the same bits (the waves' partials are added in a fixed order)
    assert torch.equal(acc, _cabi.mm_fp8_acc(ad, bd).cpu())


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("m,n,k", [(4100, 4096, 512), (4224, 4096, 256)])
def test_mm_fp8_token_tail_past_a_round_of_large_tiles(ops, fmt, m, n, k):
    """The last few rows of a block that would cost the large-tile kernel a round of their own run
    on the decode kernel in a second launch: rows either side of the seam against the oracle, per
    tensor with bias and with row / column steps."""
    from astrai_amd.extension import _cabi
    print(f"case fmt={fmt} m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m + n + k + fmt)
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    a8 = (torch.randn(m, k, generator=g) * 1.5).to(dt)
    b8 = (torch.randn(n, k, generator=g) * 1.5).to(dt)
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    sa, sb = torch.tensor([0.37]), torch.tensor([0.011])
    cut = m - m % 256
    rows = torch.cat([torch.arange(0, 5), torch.arange(cut - 6, m)])
    ad, bd = a8.to(DEV), b8.to(DEV)
    out = _cabi.mm_fp8(ad, bd, sa.to(DEV), sb.to(DEV), 0, None, bias.to(DEV))[rows.to(DEV)]
    assert_bf16_close(out, O.fp8_gemm_bias(a8[rows], b8, sa, sb, bias), what="tail rows, per tensor")
    sa_r = torch.exp2(torch.rand(m, 1, generator=g) * 6.0 - 3.0)
    sb_r = torch.exp2(torch.rand(n, generator=g) * 6.0 - 3.0)
    out = _cabi.mm_fp8(ad, bd, sa_r.to(DEV), sb_r.to(DEV), 0, None, None)[rows.to(DEV)]
    assert_bf16_close(out, O.fp8_gemm_bias(a8[rows], b8, sa_r[rows], sb_r, None), what="tail rows, row/column steps")


@pytest.mark.parametrize("m,n,k,fmt", [(3900, 4104, 1024, 0),   # even slab count: 16x16x128 instance
                                       (3900, 4104, 1152, 0),   # odd slab count: 32x32x64 instance
                                       (4097, 3848, 512, 1),    # e5m2, 16x16x128 instance
                                       (4097, 3848, 384, 1)])   # e5m2, 32x32x64 instance
def test_four_wave_kernel_both_mfma_instances_whole_output(ops, m, n, k, fmt):
    """The large-tile bf16 kernel runs on the 16x16x128 MFMA for an even number of 128-byte K
    slabs and on the 32x32x64 MFMA otherwise: ragged M and N, per-tensor steps with bias and
    row / column steps, every output against the oracle."""
    from astrai_amd.extension import _cabi
    print(f"case m={m} n={n} k={k} fmt={fmt}", flush=True)
    g = torch.Generator().manual_seed(m + n + k + fmt)
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    a8 = (torch.randn(m, k, generator=g) * 1.5).to(dt)
    b8 = (torch.randn(n, k, generator=g) * 1.5).to(dt)
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    sa, sb = torch.tensor([0.37]), torch.tensor([0.011])
    ad, bd = a8.to(DEV), b8.to(DEV)
    out = _cabi.mm_fp8(ad, bd, sa.to(DEV), sb.to(DEV), 0, None, bias.to(DEV))   # (format: the operands' dtype)
    assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa, sb, bias), what="per tensor + bias")
    sa_r = torch.exp2(torch.rand(m, 1, generator=g) * 6.0 - 3.0)
    sb_r = torch.exp2(torch.rand(n, generator=g) * 6.0 - 3.0)
    out = _cabi.mm_fp8(ad, bd, sa_r.to(DEV), sb_r.to(DEV), 0, None, None)
    assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa_r, sb_r, None), what="row/column steps")


def test_mm_fp8_rejects_bad_arguments(ops):
    a8 = torch.zeros(4, 16, dtype=torch.float8_e4m3fn, device=DEV)
    b5 = torch.zeros(4, 16, dtype=torch.float8_e5m2, device=DEV)
    one = torch.ones(1, device=DEV)
    with pytest.raises(TypeError, match="one format"):
        ops.mm_fp8(a8, b5, one, one)                       # ops/fp8.py:109-112
    with pytest.raises(RuntimeError, match="out_scale"):
        ops.mm_fp8(a8, a8, one, one, out_dtype="e4m3")     # mm.cu:158
    with pytest.raises(RuntimeError, match="float32 scalar"):
        ops.mm_fp8(a8, a8, torch.ones(2, device=DEV), one)  # mm.cu:49-54
    with pytest.raises(RuntimeError, match="inner dim"):
        ops.mm_fp8(a8, a8[:, :8].contiguous(), one, one)
    with pytest.raises(TypeError, match="bf16 tensors only"):
        ops.quantize_bf16(torch.zeros(4, device=DEV), one)


def test_config1_whole_output_at_full_size(ops):
    """BASELINE config 1 at 4096^3 with bias (seed 1): every one of the 4096 x 4096
    outputs against the oracle, so that a tile placed at the wrong coordinate, or a K
    slab dropped in one tile, cannot pass (the oracle's sgemm takes ~0.15 s)."""
    a, b, bias = O.make_inputs(1, 4096, 4096, 4096, w_std=1.0, bias=True)
    sa, sb = O.dynamic_scale(a).reshape(1), O.dynamic_scale(b).reshape(1)
    a8, _ = O.fp8_quantize(a, sa, 0)
    b8, _ = O.fp8_quantize(b, sb, 0)
    from astrai_amd.extension import _cabi
    out = _cabi.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV), 0, None, bias.to(DEV))
    want = O.fp8_gemm_bias(a8, b8, sa, sb, bias)
    assert_bf16_close(out, want, what="config1 whole output")


def test_mm_fp8_against_the_vendor_scaled_mm(ops):
    """The reference's own cross-check (tests/extension/test_fp8_mma.py:165-174): mm_fp8
    against torch._scaled_mm on a 512 x 4096 x 4096 product, atol 2 / rtol 0.01 -- and the
    same on the config-1 tensors at 4096^3, where both run their large-tile kernels."""
    from astrai_amd.extension import _cabi
    tol = golden_tol()
    torch.manual_seed(0)
    for m, n, k in [(512, 4096, 4096), (4096, 4096, 4096)]:
        print(f"case m={m} n={n} k={k}", flush=True)
        a = torch.randn(m, k, device=DEV).to(torch.bfloat16)
        b = torch.randn(n, k, device=DEV).to(torch.bfloat16)
        sa, sb = _scale(a.cpu()).to(DEV), _scale(b.cpu()).to(DEV)
        a8, _ = ops.quantize_bf16(a, sa)
        b8, _ = ops.quantize_bf16(b, sb)
        got = _cabi.mm_fp8(a8, b8, sa, sb, 0, None, None)
        try:
            ref = torch._scaled_mm(a8, b8.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
        except (RuntimeError, NotImplementedError) as e:   # no vendor fp8 GEMM on this box
            pytest.skip(f"torch._scaled_mm unavailable: {e}")
        torch.testing.assert_close(got, ref, atol=tol["atol"], rtol=tol["rtol"])
        # far tighter than the reference's gate: both are fp32 accumulations rounded once
        assert_bf16_close(got, ref.cpu(), what="vs _scaled_mm")


def golden_tol():
    from tests.conftest import load_golden
    return load_golden("reference_kats.json")["tolerances"]["vs_scaled_mm"]


@pytest.mark.parametrize("m,n,k,fmt,bias", [
    (17, 9, 33, 0, False),          # any-shape kernel (K % 16 != 0)
    (130, 200, 384, 0, True),       # small tiles
    (257, 513, 1024, 1, False),     # e5m2
    (1024, 1536, 512, 0, True),     # 128x128 tiles of the generic kernel
    (2048, 1536, 512, 1, True),     # 128x128 tiles, mid-size kernel
    (4096, 4096, 256, 0, False),    # 256x256 tiles, four-wave kernel
    (3841, 4100, 640, 0, True),     # 256x256 tiles, N % 8 != 0: ping-pong kernel
])
def test_mm_fp8_row_and_column_scales(ops, m, n, k, fmt, bias):
    """One step per activation row and per weight row: the broadcast the reference's CPU
    kernel evaluates (ops/fp8.py:118) although its CUDA binding takes scalars only."""
    from astrai_amd.extension import _cabi
    print(f"case m={m} n={n} k={k} fmt={fmt} bias={bias}", flush=True)
    g = torch.Generator().manual_seed(m + 3 * n + 7 * k)
    dt = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    a8 = (torch.randn(m, k, generator=g) * 1.5).to(dt)
    b8 = (torch.randn(n, k, generator=g) * 1.5).to(dt)
    sa = torch.exp2(torch.rand(m, 1, generator=g) * 6.0 - 3.0)
    sb = torch.exp2(torch.rand(n, generator=g) * 6.0 - 3.0)
    bvec = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    out = _cabi.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV), 0, None,
                       bvec.to(DEV) if bias else None)
    assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa, sb, bvec), what="row/column scales")
    # through the dispatcher op, and with only one of the two per row
    out = ops.mm_fp8(a8.to(DEV), b8.to(DEV), sa[:1, 0].to(DEV), sb.reshape(1, n).to(DEV))
    assert_bf16_close(out, O.fp8_gemm(a8, b8, sa[:1, 0], sb.reshape(1, n)), what="column scales only")


def test_empty_operands(ops):
    """No rows, no columns, no elements: shapes and dtypes as for any other input,
    no launch, no error (the reference allocates the same empty outputs, mm.cu:111-124,154-160)."""
    from astrai_amd.extension import _cabi
    s = torch.ones(1, device=DEV)
    x8, amax = ops.quantize_bf16(torch.empty(0, 64, device=DEV, dtype=torch.bfloat16), s)
    assert x8.shape == (0, 64) and x8.dtype == torch.float8_e4m3fn and amax.shape == (1,) and float(amax) == 0.0
    a8 = torch.zeros(0, 64, device=DEV).to(torch.float8_e4m3fn)
    b8 = torch.zeros(24, 64, device=DEV).to(torch.float8_e4m3fn)
    out = ops.mm_fp8(a8, b8, s, s)
    assert out.shape == (0, 24) and out.dtype == torch.bfloat16
    out = ops.mm_fp8(b8, a8, s, s)
    assert out.shape == (24, 0)
    y, ax, aw = _cabi.linear_forward_fp8(torch.empty(2, 0, 64, device=DEV, dtype=torch.bfloat16),
                                         torch.randn(24, 64, device=DEV).to(torch.bfloat16), None, s, s)
    assert y.shape == (2, 0, 24) and float(ax) == 0.0 and float(aw) > 0.0
    xq, sx = _cabi.quantize_int8_rows(torch.empty(0, 128, device=DEV, dtype=torch.bfloat16))
    assert xq.shape == (0, 128) and sx.numel() == 0
    acc = _cabi.mm_int8(torch.empty(0, 128, device=DEV, dtype=torch.int8),
                        torch.zeros(16, 128, device=DEV, dtype=torch.int8), None, None, None, 2)
    assert acc.shape == (0, 16) and acc.dtype == torch.int32


def test_random_shape_sweep_fp8(ops):
    """Forty seeded random shapes, both formats, through the default dispatch."""
    g = torch.Generator().manual_seed(777)
    for i in range(40):
        m = int(torch.randint(1, 400, (1,), generator=g))
        n = int(torch.randint(1, 600, (1,), generator=g))
        k = int(torch.randint(1, 1500, (1,), generator=g))
        fmt = torch.float8_e5m2 if i % 4 == 3 else torch.float8_e4m3fn
        print(f"case {i}: m={m} n={n} k={k} {fmt}", flush=True)
        a8 = (torch.randn(m, k, generator=g) * 1.5).to(fmt)
        b8 = (torch.randn(n, k, generator=g) * 1.5).to(fmt)
        sa = torch.rand(1, generator=g) + 0.25
        sb = torch.rand(1, generator=g) + 0.25
        out = ops.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
        assert_bf16_close(out, O.fp8_gemm(a8, b8, sa, sb), what=f"sweep {m}x{n}x{k}")


# ---- 128-block scaled ----

@pytest.mark.parametrize("m,n,k", [(3, 130, 256), (64, 128, 128), (130, 200, 384), (257, 513, 1024)])
def test_block128_gemm_small(m, n, k):
    from astrai_amd.extension.ops import fp8_block as blk
    print(f"case m={m} n={n} k={k}", flush=True)
    x, w, _ = O.make_inputs(3, m, n, k, outlier_p=0.01)
    x8, sa = O.fp8_quantize_act_block128(x)
    w8, sb = O.fp8_quantize_weight_block128(w)
    out = blk.mm_fp8_blockscaled(x8.to(DEV), w8.to(DEV), sa.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm_blockscaled(x8, w8, sa, sb), what="block128")


@pytest.mark.parametrize("m,n,k,bias", [(1, 2048, 7168, False), (16, 2048, 7168, True), (64, 11008, 4096, False),
                                        (33, 130, 256, True), (4, 7168, 2048, False), (48, 1001, 512, True),
                                        (7, 2052, 5632, False)])
def test_block128_decode_shapes_row_range_kernel(m, n, k, bias):
    """At most 64 activation rows with K % 256 == 0: the block-scaled instance of the row-range
    decode kernel (each 128-byte half of an item is one K-block, scaled before it is accumulated),
    wide scale ranges (outliers in 1% of the weights), ragged N, weight blocks cut by workgroup ranges."""
    from astrai_amd.extension.ops import fp8_block as blk
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    x, w, b = O.make_inputs(3, m, n, k, outlier_p=0.01, bias=bias)
    x8, sa = O.fp8_quantize_act_block128(x)
    w8, sb = O.fp8_quantize_weight_block128(w)
    bd = b.to(DEV) if bias else None
    out = blk.mm_fp8_blockscaled(x8.to(DEV), w8.to(DEV), sa.to(DEV), sb.to(DEV), bd)
    assert_bf16_close(out, O.fp8_gemm_blockscaled(x8, w8, sa, sb, b if bias else None), what="block128 decode rows")
    again = blk.mm_fp8_blockscaled(x8.to(DEV), w8.to(DEV), sa.to(DEV), sb.to(DEV), bd)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))    # fixed summation order


@pytest.mark.parametrize("m,n,k,bias", [(1536, 1536, 512, False), (1100, 2050, 384, True), (2048, 1280, 1024, True),
                                        (1793, 1798, 256, False)])
def test_block128_mid_size_tiles(m, n, k, bias):
    """Shapes with at least 140 tiles of 128 x 128 but too few of 256 x 256: the block-scaled instance of
    the mid-size kernel (a slab = one K-block, scaled before it joins the accumulator); ragged rows
    and columns, outliers in 1% of the weights for a wide scale range."""
    from astrai_amd.extension.ops import fp8_block as blk
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    x, w, b = O.make_inputs(3, m, n, k, outlier_p=0.01, bias=bias)
    x8, sa = O.fp8_quantize_act_block128(x)
    w8, sb = O.fp8_quantize_weight_block128(w)
    out = blk.mm_fp8_blockscaled(x8.to(DEV), w8.to(DEV), sa.to(DEV), sb.to(DEV), b.to(DEV) if bias else None)
    assert_bf16_close(out, O.fp8_gemm_blockscaled(x8, w8, sa, sb, b if bias else None), what="block128 mid-size")


@pytest.mark.parametrize("m,n,k,bias", [(130, 200, 384, True), (300, 520, 1152, False), (256, 2048, 5632, True),
                                        (65, 778, 128, False), (1000, 1024, 2048, True)])
def test_block128_small_tiles(m, n, k, bias):
    """Fewer than 140 tiles of 128 x 128 (and more rows than the decode kernel takes): the block-scaled
    instance of the 64 x 64-tile kernel (ring of stages, a slab = one K-block scaled before it joins the
    accumulator, its steps requested a slab ahead); ragged rows and columns, one to 44 slabs, wide scale range."""
    from astrai_amd.extension import _cabi
    from astrai_amd.extension.ops import fp8_block as blk
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    x, w, b = O.make_inputs(3, m, n, k, outlier_p=0.01, bias=bias)
    x8, sa = O.fp8_quantize_act_block128(x)
    w8, sb = O.fp8_quantize_weight_block128(w)
    out = blk.mm_fp8_blockscaled(x8.to(DEV), w8.to(DEV), sa.to(DEV), sb.to(DEV), b.to(DEV) if bias else None)
    assert _cabi.last_kernel() == "small64", _cabi.last_kernel()
    assert_bf16_close(out, O.fp8_gemm_blockscaled(x8, w8, sa, sb, b if bias else None), what="block128 small tiles")


def test_block128_golden_exact_rationals(golden):
    from astrai_amd.extension.ops import fp8_block as blk
    for c in golden("fp8_gemm_small.json")["block128"]:
        a8 = torch.tensor(c["a"], dtype=torch.uint8).view(torch.float8_e4m3fn)
        b8 = torch.tensor(c["b"], dtype=torch.uint8).view(torch.float8_e4m3fn)
        sa, sb = torch.tensor(c["sa"]), torch.tensor(c["sb"])
        exact = torch.tensor(c["exact"], dtype=torch.float64)
        out = blk.mm_fp8_blockscaled(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
        assert_bf16_close(out, exact.to(torch.bfloat16), what="block128 exact")


def test_block128_reduces_to_per_tensor(ops):
    from astrai_amd.extension.ops import fp8_block as blk
    x, w, _ = O.make_inputs(4, 96, 300, 512, w_std=1.0)
    s = torch.tensor([0.03125])
    a8, _ = O.fp8_quantize_saturating(x, s, 0)
    b8, _ = O.fp8_quantize_saturating(w, s, 0)
    sa = torch.full((96, 4), 0.03125)
    sb = torch.full((3, 4), 0.03125)
    got = blk.mm_fp8_blockscaled(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
    want = ops.mm_fp8(a8.to(DEV), b8.to(DEV), s.to(DEV), s.to(DEV))
    assert_bf16_close(got, want.cpu(), what="block==tensor")


def test_config3_shape_whole_output():
    """BASELINE config 3 (seed 3): A[8192,7168], B[2048,7168] with 1% x20 outliers,
    quantized on the device, GEMM on the device; codes, steps and every one of the
    8192 x 2048 outputs against the oracle (~0.4 s of CPU)."""
    from astrai_amd.extension.ops import fp8_block as blk
    x, w, _ = O.make_inputs(3, 8192, 2048, 7168, outlier_p=0.01)
    x8, sa = blk.quantize_act_block128(x.to(DEV))
    w8, sb = blk.quantize_weight_block128(w.to(DEV))
    out = blk.mm_fp8_blockscaled(x8, w8, sa, sb)
    rx8, rsa = O.fp8_quantize_act_block128(x)
    rw8, rsb = O.fp8_quantize_weight_block128(w)
    assert torch.equal(x8.cpu().view(torch.uint8), rx8.view(torch.uint8))
    assert torch.equal(w8.cpu().view(torch.uint8), rw8.view(torch.uint8))
    assert torch.equal(sa.cpu(), rsa) and torch.equal(sb.cpu(), rsb)
    assert_bf16_close(out, O.fp8_gemm_blockscaled(rx8, rw8, rsa, rsb), what="config3 whole output")


@pytest.mark.parametrize("m,n,k", [(3841, 3336, 256),    # two slabs: the shortest K the large kernel takes
                                   (4000, 3592, 384),    # three slabs
                                   (3600, 4096, 1152)])
def test_block128_large_kernel_wide_scale_range(m, n, k):
    """The 256x256-tile block-scaled kernel (>= 192 tiles, N % 8 == 0) on ragged M and
    N, with block scales spread over twelve octaves so that every slab's rescaling
    factor matters, checked on the whole output."""
    from astrai_amd.extension.ops import fp8_block as blk
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m + n + k)
    a8 = (torch.randn(m, k, generator=g) * 2.0).to(torch.float8_e4m3fn)
    b8 = (torch.randn(n, k, generator=g) * 2.0).to(torch.float8_e4m3fn)
    sa = torch.exp2(torch.rand(m, k // 128, generator=g) * 12.0 - 6.0)
    sb = torch.exp2(torch.rand((n + 127) // 128, k // 128, generator=g) * 12.0 - 6.0)
    out = blk.mm_fp8_blockscaled(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
    assert_bf16_close(out, O.fp8_gemm_blockscaled(a8, b8, sa, sb), what="block128 large")


# ---- large ragged shapes: the 256x256-tile kernels with partial edge tiles ----

@pytest.mark.parametrize("m,n,k,bias", [(3900, 4104, 1152, True),    # N % 8 == 0: four-wave kernel
                                        (3841, 4100, 640, False),   # N % 8 != 0: ping-pong kernel
                                        (4096, 3848, 256, False),   # shortest K the big kernels take
                                        (1700, 2056, 384, True),    # 14 x 17 tiles of 128 x 128: mid-size kernel
                                        (1793, 1798, 256, False),   # the same, N % 4 != 0: element stores
                                        (2048, 2048, 2048, False)])
def test_large_ragged_tiles_with_guard_rows(m, n, k, bias):
    """Edge tiles of the large-shape kernels: rows past M / columns past N must
    read as zero and must not be written. The call goes through the C ABI into
    an output buffer with sentinel rows behind row M-1."""
    from astrai_amd.extension import _cabi
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    lib = _cabi.load()
    g = torch.Generator().manual_seed(m + n + k)
    a8 = (torch.randn(m, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    b8 = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    bvec = torch.randn(n, generator=g).to(torch.bfloat16) if bias else None
    sa, sb = torch.tensor([0.75]), torch.tensor([1.25])
    guard = 8
    out = torch.full((m + guard, n), -777.0, dtype=torch.bfloat16, device=DEV)
    da, db, dsa, dsb = a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV)
    dbias = bvec.to(DEV) if bias else None
    rc = lib.astrai_w8a8_gemm_fp8_pt(da.data_ptr(), db.data_ptr(), dsa.data_ptr(), dsb.data_ptr(), None,
                                     dbias.data_ptr() if bias else None, out.data_ptr(), m, n, k, 0, 0,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.astrai_w8a8_last_error()
    torch.cuda.synchronize()
    assert torch.all(out[m:] == -777.0), "rows past M were written"
    rows = torch.cat([torch.arange(0, 3), torch.arange(255, 258), torch.arange(m - 3, m)])
    want = O.fp8_gemm_bias(a8[rows], b8, sa, sb, bvec)
    assert_bf16_close(out[rows], want, what="ragged rows")
    cols = torch.cat([torch.arange(0, 2), torch.arange(n - 9, n)])
    want_c = O.fp8_gemm_bias(a8, b8[cols], sa, sb, bvec[cols] if bias else None)
    assert_bf16_close(out[:m, cols], want_c, what="ragged columns")


def test_block128_random_shape_sweep():
    """Seeded random shapes of the block-scaled GEMM, small tiles to the 256x256-tile kernel,
    ragged M and N, scales over eight octaves, whole output against the oracle."""
    from astrai_amd.extension.ops import fp8_block as blk
    g = torch.Generator().manual_seed(909)
    r = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    shapes = [(r(1, 600), r(1, 700), 128 * r(1, 9)) for _ in range(12)]
    shapes += [(r(3500, 4200), 8 * r(430, 520), 128 * r(2, 5)) for _ in range(3)]   # >= 192 tiles of 256^2
    for (m, n, k) in shapes:
        print(f"case m={m} n={n} k={k}", flush=True)
        a8 = (torch.randn(m, k, generator=g) * 2.0).to(torch.float8_e4m3fn)
        b8 = (torch.randn(n, k, generator=g) * 2.0).to(torch.float8_e4m3fn)
        sa = torch.exp2(torch.rand(m, k // 128, generator=g) * 8.0 - 4.0)
        sb = torch.exp2(torch.rand((n + 127) // 128, k // 128, generator=g) * 8.0 - 4.0)
        out = blk.mm_fp8_blockscaled(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV))
        assert_bf16_close(out, O.fp8_gemm_blockscaled(a8, b8, sa, sb), what=f"block128 {m}x{n}x{k}")


def test_linear_forward_backward_random_shape_sweep(ops):
    """Twelve seeded random layer shapes through the fused forward and the backward (all three
    gradients), bias in every other case, against the oracle's codes."""
    g = torch.Generator().manual_seed(2025)
    r = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for i in range(12):
        m, n, k = r(1, 300), r(1, 300), r(1, 500)
        print(f"case {i}: m={m} n={n} k={k}", flush=True)
        x = torch.randn(m, k, generator=g).to(torch.bfloat16)
        w = torch.randn(n, k, generator=g).to(torch.bfloat16)
        gr = torch.randn(m, n, generator=g).to(torch.bfloat16)
        bias = torch.randn(n, generator=g).to(torch.bfloat16) if i % 2 else None
        sx, sw, sg = _scale(x), _scale(w), _scale(gr)
        out, ax, aw = ops.linear_forward_fp8(x.to(DEV), w.to(DEV), bias.to(DEV) if i % 2 else None,
                                             sx.to(DEV), sw.to(DEV))
        want, wax, waw = O.linear_forward_fp8(x, w, bias, sx, sw)
        assert_bf16_close(out, want, what=f"forward {m}x{n}x{k}")
        assert ax.item() == wax.item() and aw.item() == waw.item()
        gx, gw, gb, amax_g = ops.linear_backward_fp8(
            gr.to(DEV), x.to(DEV), w.to(DEV), [1, 1, 1], sg.to(DEV), sw.to(DEV), sx.to(DEV), "e4m3")
        qg = O.fp8_quantize(gr, sg, 0)[0].float()
        qw = O.fp8_quantize(w, sw, 0)[0].float()
        qx = O.fp8_quantize(x, sx, 0)[0].float()
        assert_bf16_close(gx, (qg @ qw * sg * sw).to(torch.bfloat16), what=f"dX {m}x{n}x{k}")
        assert_bf16_close(gw, (qg.t() @ qx * sg * sx).to(torch.bfloat16), what=f"dW {m}x{n}x{k}")
        torch.testing.assert_close(gb.cpu(), gr.sum(0).to(torch.bfloat16))
        assert amax_g.item() == gr.abs().max().item()


@pytest.mark.parametrize("m,n,k", [(256, 256, 4096),     # generic tiled kernel (16x16x128 MFMA)
                                   (4096, 4096, 1024)])  # large-tile kernel (32x32x64 MFMA)
def test_fp8_mfma_accumulator_deviation_from_exact_sum(m, n, k):
    """How far the fp8 MFMA's fp32 accumulator sits from the exact sum of the (exactly
    representable) products, measured rather than asserted: relative to sum |a_k b_k| the
    deviation stays below 2^-17 per element with an rms below 2^-19 (measured max / rms: 1.6e-6 /
    3.7e-7 with the 16x16x128 instruction at K = 4096, 4.0e-6 / 7.3e-7 with the 32x32x64 one at
    K = 1024) -- more than the 6e-8 of one fp32 rounding, i.e. the instructions do not keep every
    product bit while they add, and far inside the 2^-8 of the bf16 output. Relative to the rms
    of the results it stays below 2e-4 (measured 6.4e-5 / 8.3e-5)."""
    from astrai_amd.extension import _cabi
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m + k)
    a8 = (torch.randn(m, k, generator=g) * 30.0).clamp(-448, 448).to(torch.float8_e4m3fn)
    b8 = (torch.randn(n, k, generator=g) * 30.0).clamp(-448, 448).to(torch.float8_e4m3fn)
    acc = _cabi.mm_fp8_acc(a8.to(DEV), b8.to(DEV)).cpu()
    rows = torch.arange(0, m, max(1, m // 128))          # float64 reference on sampled rows
    exact = a8[rows].double() @ b8.double().t()
    mass = a8[rows].double().abs() @ b8.double().abs().t()
    rel = (acc[rows].double() - exact).abs() / mass
    vs_result = ((acc[rows].double() - exact).abs().max() / exact.pow(2).mean().sqrt()).item()
    print(f"max {rel.max().item():.3g} rms {rel.pow(2).mean().sqrt().item():.3g} "
          f"max against the results' rms {vs_result:.3g}", flush=True)
    assert rel.max().item() < 2.0 ** -17
    assert rel.pow(2).mean().sqrt().item() < 2.0 ** -19
    assert vs_result < 2e-4


def test_graph_replay_of_decode_and_two_launch_products_equals_eager():
    """The fp8 decode kernels (per-tensor and 128-block steps) and a product that runs as two
    launches (large tiles + a token tail on the decode kernel), captured in one graph: every
    replay, with eager work and new inputs in between, gives the eager call's bits."""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(77)
    w8 = (torch.randn(3072, 2048, generator=g) * 1.5).to(torch.float8_e4m3fn).to(DEV)
    x8 = (torch.randn(8, 2048, generator=g) * 1.5).to(torch.float8_e4m3fn).to(DEV)
    sa, sb = torch.tensor([0.3], device=DEV), torch.tensor([0.02], device=DEV)
    xb = torch.randn(16, 2048, generator=g).to(torch.bfloat16).to(DEV)
    wb8, sbb = _cabi.quantize_fp8_block128_weight((torch.randn(1024, 2048, generator=g) * 0.02).to(torch.bfloat16).to(DEV))
    big = torch.randint(-127, 128, (4100, 512), generator=g, dtype=torch.int8).to(DEV)
    wbig = torch.randint(-127, 128, (4096, 512), generator=g, dtype=torch.int8).to(DEV)
    sbig, swbig = (torch.rand(4100, generator=g) * 0.01).to(DEV), (torch.rand(4096, generator=g) * 0.01).to(DEV)

    def run():
        xb8, sab = _cabi.quantize_fp8_block128_act(xb)
        return (_cabi.mm_fp8(x8, w8, sa, sb), _cabi.mm_fp8_block128(xb8, wb8, sab, sbb),
                _cabi.mm_int8(big, wbig, sbig, swbig))

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            run()
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run()
    for i in range(3):
        x8.copy_((torch.randn(8, 2048, generator=g) * 1.5).to(torch.float8_e4m3fn))
        xb.copy_(torch.randn(16, 2048, generator=g).to(torch.bfloat16))
        big.copy_(torch.randint(-127, 128, (4100, 512), generator=g, dtype=torch.int8))
        graph.replay()
        torch.cuda.synchronize()
        want = run()
        for got, ref in zip(outs, want):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), i
