"""int8 W8A8 kernels vs the oracle: int32 accumulators bit-exact, bf16 outputs
within 1e-2 relative after the scaled epilogue (HIP path through the C ABI)."""

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


def _rand_i8(g, *shape):
    return torch.randint(-127, 128, shape, generator=g, dtype=torch.int8)


RAGGED = [(16, 8, 32), (17, 9, 33), (31, 15, 64), (32, 48, 96), (19, 13, 37), (1, 1, 1), (3, 5, 7)]
TILE_EDGES = [(64, 64, 128), (65, 63, 144), (128, 128, 256), (129, 257, 272), (256, 256, 512),
              (300, 500, 1040), (511, 513, 2048), (1024, 768, 1024)]


@pytest.mark.parametrize("m,n,k", RAGGED + TILE_EDGES)
def test_int32_accumulator_bit_exact(C, m, n, k):
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m * 7 + n * 3 + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    got = C.mm_int8(a.to(DEV), b.to(DEV), None, None, None, 2).cpu()
    assert got.dtype == torch.int32 and torch.equal(got, O.int8_acc(a, b))


def test_random_shape_sweep_default_dispatch_bit_exact(C):
    """Sixty seeded random shapes through the default entry point, whichever kernel
    it picks (single-token, row-range, tiled, generic): accumulators bit-exact, and the
    scaled bf16 output bit-equal to the oracle's elementwise epilogue."""
    g = torch.Generator().manual_seed(20240)
    for i in range(60):
        m = int(torch.randint(1, 301, (1,), generator=g))
        n = int(torch.randint(1, 701, (1,), generator=g))
        k = int(torch.randint(1, 1201, (1,), generator=g))
        if i % 3 == 0:
            k = (k + 255) // 256 * 256   # the decode kernels need K % 256 == 0
        if i % 4 == 0:
            m = 1 + i % 40
        print(f"case {i}: m={m} n={n} k={k}", flush=True)
        a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
        want = O.int8_acc(a, b)
        got = C.mm_int8(a.to(DEV), b.to(DEV), None, None, None, 2).cpu()
        assert torch.equal(got, want), (m, n, k)
        sa = torch.rand(m, generator=g) * 0.02 + 0.001
        sb = torch.rand(n, generator=g) * 0.02 + 0.001
        out = C.mm_int8(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV), None, 0).cpu()
        ref = (want.float() * sa[:, None] * sb[None, :]).to(torch.bfloat16)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), (m, n, k)
        # the same product joined to a residual stream in the epilogue (or by the addition pass)
        r = (torch.randn(m, n, generator=g) * float(ref.float().abs().mean() + 1e-3)).to(torch.bfloat16)
        fused = C.mm_int8_resid(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV), r.to(DEV)).cpu()
        assert torch.equal(fused.view(torch.int16), (ref + r).view(torch.int16)), (m, n, k)


@pytest.mark.parametrize("m,n,k", [(300, 520, 1032), (64, 1024, 1288), (1, 2048, 8200), (513, 257, 2047)])
def test_k_not_in_16_byte_pieces_zero_padded_bit_exact(C, m, n, k):
    """K % 16 != 0 on a product large enough for the wrapper to zero-pad the rows for the tuned
    kernels: accumulators, the scaled output and the residual form stay bit-exact, and the
    caller's tensors are untouched."""
    print(f"case m={m} n={n} k={k}", flush=True)
    assert k % 16 and m * n * k >= C._PAD_K_MIN_MACS
    g = torch.Generator().manual_seed(m + n + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    ad, bd = a.to(DEV), b.to(DEV)
    padded = C._pad_k(ad, bd)
    assert padded[2] % 128 == 0 and padded[0].shape == (m, padded[2]) and padded[1].shape == (n, padded[2])
    assert torch.equal(padded[0][:, :k], ad) and not padded[0][:, k:].any() and not padded[1][:, k:].any()
    want = O.int8_acc(a, b)
    assert torch.equal(C.mm_int8(ad, bd, None, None, None, 2).cpu(), want)
    sa = torch.rand(m, generator=g) * 0.02 + 0.001
    sb = torch.rand(n, generator=g) * 0.02 + 0.001
    ref = (want.float() * sa[:, None] * sb[None, :]).to(torch.bfloat16)
    out = C.mm_int8(ad, bd, sa.to(DEV), sb.to(DEV), None, 0).cpu()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    r = torch.randn(m, n, generator=g).to(torch.bfloat16)
    fused = C.mm_int8_resid(ad, bd, sa.to(DEV), sb.to(DEV), r.to(DEV)).cpu()
    assert torch.equal(fused.view(torch.int16), (ref + r).view(torch.int16))
    assert torch.equal(ad.cpu(), a) and torch.equal(bd.cpu(), b)


@pytest.mark.parametrize("m,n,k", [(4100, 4096, 512), (4224, 4096, 256), (4097, 4104, 768), (8200, 2048, 512)])
def test_token_tail_past_a_round_of_large_tiles_bit_exact(C, m, n, k):
    """A few rows more than whole 256-row tiles that would cost the large-tile kernel a round of
    their own go to the decode kernel in a second launch: the seam must not show -- bf16 output
    bit-equal to the oracle's epilogue on sampled rows either side of it, with bias and as the
    residual form."""
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m + n + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    sa = torch.rand(m, generator=g) * 0.02 + 0.001
    sb = torch.rand(n, generator=g) * 0.02 + 0.001
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    cut = m - m % 256
    rows = torch.cat([torch.arange(0, 5), torch.arange(cut - 6, m)])
    acc = O.int8_acc(a[rows], b).float()
    ad, bd, sad, sbd = a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV)
    out = C.mm_int8(ad, bd, sad, sbd, None, 0)[rows.to(DEV)].cpu()
    ref = (acc * sa[rows, None] * sb[None, :]).to(torch.bfloat16)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    out = C.mm_int8(ad, bd, sad, sbd, bias.to(DEV), 0)[rows.to(DEV)].cpu()
    refb = (acc * sa[rows, None] * sb[None, :] + bias.float()).to(torch.bfloat16)
    assert torch.equal(out.view(torch.int16), refb.view(torch.int16))
    r = torch.randn(m, n, generator=g).to(torch.bfloat16)
    fused = C.mm_int8_resid(ad, bd, sad, sbd, r.to(DEV))[rows.to(DEV)].cpu()
    assert torch.equal(fused.view(torch.int16), (ref + r[rows]).view(torch.int16))
    # the entry that names the tiled kernels runs the whole product on them: the same bits
    tiled = C.mm_int8(ad, bd, sad, sbd, None, 0, kernel="tiled")[rows.to(DEV)].cpu()
    assert torch.equal(tiled.view(torch.int16), ref.view(torch.int16))


def test_golden_integer_cases_including_worst_case_magnitude(C, golden):
    for c in golden("int8_small.json")["gemm"]:
        a = torch.tensor(c["a"], dtype=torch.int8)
        b = torch.tensor(c["b"], dtype=torch.int8)
        want = torch.tensor(c["acc"], dtype=torch.int32)
        for kernel in ("auto", "tiled") if c["k"] % 16 == 0 else ("auto",):
            got = C.mm_int8(a.to(DEV), b.to(DEV), None, None, None, 2, kernel).cpu()
            assert torch.equal(got, want), (c["m"], c["n"], c["k"], kernel)


@pytest.mark.parametrize("kernel", ["tiled", "gemv"])
@pytest.mark.parametrize("m", [1, 2, 4, 16, 17, 33, 64, 65, 100, 128])
@pytest.mark.parametrize("n,k", [(11008, 4096), (1000, 512), (40, 256), (3072, 2048), (2048, 5632), (200, 11008),
                                 # row ranges of 17..32 and 33..48 rows, ragged N
                                 (8192, 512), (5000, 256), (10001, 768)])
def test_skinny_shapes_both_kernels_bit_exact(C, kernel, m, n, k):
    """Decode shapes through the wave-split row-range kernel and through the tiled
    kernel: the split-K integer sums must equal the single-pass ones."""
    print(f"case kernel={kernel} m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m + n + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    got = C.mm_int8(a.to(DEV), b.to(DEV), None, None, None, 2, kernel).cpu()
    assert torch.equal(got, O.int8_acc(a, b))


@pytest.mark.parametrize("m,n,k", [(2, 11008, 4096), (32, 3072, 2048), (48, 11264, 2048), (128, 2048, 5632),
                                   (5, 1001, 768), (64, 11008, 4096), (64, 8192, 512), (40, 10001, 768),
                                   (33, 5000, 256)])
def test_skinny_bf16_epilogue_bit_exact(C, m, n, k):
    """The row-range kernel's dequant epilogue (scales, bias, one rounding; ragged N
    takes the scalar stores) against the oracle's elementwise fp32 formula."""
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m * 7 + n + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    sa = torch.rand(m, generator=g) * 0.02 + 0.001
    sb = torch.rand(n, generator=g) * 0.02 + 0.001
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    got = C.mm_int8(a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV), bias.to(DEV), 0, "gemv").cpu()
    want = O.int8_gemm(a, b, sa, sb, bias)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_gemv_entry_rejects_what_it_cannot_run(C):
    a = torch.zeros(129, 256, dtype=torch.int8, device=DEV)
    b = torch.zeros(8, 256, dtype=torch.int8, device=DEV)
    with pytest.raises(RuntimeError, match="M <= 128"):
        C.mm_int8(a, b, None, None, None, 2, "gemv")
    with pytest.raises(RuntimeError, match="multiple of 256"):
        C.mm_int8(a[:4, :128].contiguous(), b[:, :128].contiguous(), None, None, None, 2, "gemv")
    with pytest.raises(RuntimeError, match="int8"):
        C.mm_int8(a.float(), b, None, None, None, 2)
    with pytest.raises(RuntimeError, match="inner dim"):
        C.mm_int8(a, b[:, :128].contiguous(), None, None, None, 2)


@pytest.mark.parametrize("m,n,k,bias", [(16, 2048, 2048, False), (16, 2048, 2048, True),
                                        (17, 9, 33, True), (300, 500, 1040, True),
                                        (64, 11008, 4096, False), (1, 11008, 4096, True)])
def test_config0_scheme_bf16_epilogue(C, m, n, k, bias):
    """BASELINE config 0 (seed 0: X[16,2048]~N(0,1) per-token, W[2048,2048]~N(0,.02)
    per-channel) and neighbours: quantized by the oracle, multiplied by the kernel."""
    print(f"case m={m} n={n} k={k} bias={bias}", flush=True)
    x, w, b = O.make_inputs(0, m, n, k, bias=bias)
    xq, sx = O.int8_quantize_rows(x)
    wq, sw = O.int8_quantize_rows(w)
    want = O.int8_gemm(xq, wq, sx, sw, b)
    got = C.mm_int8(xq.to(DEV), wq.to(DEV), sx.to(DEV), sw.reshape(-1).to(DEV),
                    b.to(DEV) if bias else None, 0)
    assert got.dtype == torch.bfloat16
    assert_bf16_close(got, want, what=f"int8 {m}x{n}x{k}")
    # the epilogue is elementwise fp32 on an exact integer: expect bit equality
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


def test_linear_forward_int8_end_to_end_matches_oracle(C):
    from astrai_amd.extension.ops import int8 as ops
    x, w, b = O.make_inputs(2, 4, 11008, 4096, bias=True)
    wq_d, sw_d = ops.quantize_int8_per_channel(w.to(DEV))
    wq, sw = O.int8_quantize_rows(w)
    assert torch.equal(wq_d.cpu(), wq) and torch.equal(sw_d.cpu(), sw.reshape(-1))
    x3 = x.reshape(2, 2, 4096)
    got = ops.linear_forward_int8(x3.to(DEV), wq_d, sw_d, b.to(DEV))
    want = O.int8_linear(x3, wq, sw, b)
    assert got.shape == (2, 2, 11008)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


def test_full_size_linearity_property(C):
    """4096^3: every one of the 4096 x 4096 int32 accumulators against the exact oracle
    (all 16 x 16 tiles of the launch, so a tile at a wrong coordinate or a K slab dropped
    in one tile fails), and exactness of the integer ring on top --
    acc(a1+a2, b) == acc(a1, b) + acc(a2, b) with operands kept inside int8."""
    g = torch.Generator().manual_seed(5)
    m = n = k = 4096
    a1 = torch.randint(-63, 64, (m, k), generator=g, dtype=torch.int8)
    a2 = torch.randint(-63, 64, (m, k), generator=g, dtype=torch.int8)
    b = _rand_i8(g, n, k)
    bd = b.to(DEV)
    s = C.mm_int8((a1 + a2).to(DEV), bd, None, None, None, 2, "tiled")
    p1 = C.mm_int8(a1.to(DEV), bd, None, None, None, 2, "tiled")
    p2 = C.mm_int8(a2.to(DEV), bd, None, None, None, 2, "tiled")
    assert torch.equal(s, p1 + p2)
    assert torch.equal(p1.cpu(), O.int8_acc(a1, b))
    # the bf16 epilogue of the four-wave kernel on the same product, every element
    sx = torch.rand(m, generator=g) + 0.5
    sw = (torch.rand(n, generator=g) + 0.5) * 1e-3
    y = C.mm_int8(a1.to(DEV), bd, sx.to(DEV), sw.to(DEV), None, 0, "tiled")
    assert torch.equal(y.cpu().view(torch.int16), O.int8_gemm(a1, b, sx, sw).view(torch.int16))


@pytest.mark.parametrize("m,n,k,out_dtype", [(3900, 4104, 1152, 0),   # bf16, N % 8 == 0: four-wave kernel
                                             (3841, 4100, 640, 0),    # bf16, N % 8 != 0: ping-pong kernel
                                             (3900, 4104, 384, 2),    # int32 accumulator: ping-pong kernel
                                             (1700, 2052, 384, 0),    # 14 x 17 tiles of 128 x 128: mid-size kernel
                                             (1793, 1798, 256, 0),    # the same, N % 4 != 0: element stores
                                             (2048, 3072, 2048, 0),   # a 2048-token block of the config-4 q|k|v projection
                                             (512, 11264, 2048, 0)])  # a 512-token block of its gate|up projection (4 x 88 tiles)
def test_large_ragged_tiles_with_guard_rows(C, m, n, k, out_dtype):
    """Edge tiles of the large-shape kernels: bit-exact int32 (or the bf16
    epilogue of it) on the first / tile-boundary / last rows and the last columns,
    and nothing written behind row M-1 (sentinel rows after the output)."""
    print(f"case m={m} n={n} k={k} out_dtype={out_dtype}", flush=True)
    lib = C.load()
    g = torch.Generator().manual_seed(m + n + k)
    a = _rand_i8(g, m, k)
    b = _rand_i8(g, n, k)
    sa = torch.rand(m, generator=g) * 0.02 + 0.001
    sb = torch.rand(n, generator=g) * 0.02 + 0.001
    guard = 8
    if out_dtype == 2:
        out = torch.full((m + guard, n), -777, dtype=torch.int32, device=DEV)
    else:
        out = torch.full((m + guard, n), -777.0, dtype=torch.bfloat16, device=DEV)
    da, db, dsa, dsb = a.to(DEV), b.to(DEV), sa.to(DEV), sb.to(DEV)
    rc = lib.astrai_w8a8_gemm_int8_ptpc(da.data_ptr(), db.data_ptr(), dsa.data_ptr(), dsb.data_ptr(), None,
                                        out.data_ptr(), m, n, k, out_dtype,
                                        torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.astrai_w8a8_last_error()
    torch.cuda.synchronize()
    assert torch.all(out[m:] == -777), "rows past M were written"
    rows = torch.cat([torch.arange(0, 3), torch.arange(255, 258), torch.arange(m - 3, m)])
    cols = torch.cat([torch.arange(0, 2), torch.arange(n - 9, n)])
    if out_dtype == 2:
        assert torch.equal(out[rows].cpu(), O.int8_acc(a[rows], b))
        assert torch.equal(out[:m, cols].cpu(), O.int8_acc(a, b[cols]))
    else:
        assert torch.equal(out[rows].cpu(), O.int8_gemm(a[rows], b, sa[rows], sb))
        assert torch.equal(out[:m, cols].cpu(), O.int8_gemm(a, b[cols], sa, sb[cols]))


SMALL_TILE_SHAPES = [(64, 64, 128),        # one tile, one slab
                     (130, 200, 384),      # three slabs: fewer than the ring's stages
                     (129, 257, 512),      # ragged rows and columns in the edge tiles
                     (256, 4096, 4096),    # one workgroup per compute unit, 32 slabs
                     (384, 2048, 5632),    # 44 slabs
                     (300, 778, 1152),     # odd slab count, N % 4 != 0: scalar stores
                     (1000, 2048, 2048),   # two workgroups per compute unit
                     (64, 2048, 2176)]     # few rows with a K the decode kernels do not take


@pytest.mark.parametrize("m,n,k", SMALL_TILE_SHAPES)
def test_small_tile_kernel_int8_and_fp8(C, m, n, k):
    """Shapes with too few 128 x 128 tiles for the mid-size kernel and K in whole 128-byte slabs run
    64 x 64 tiles fed by a ring of direct-to-LDS stages: bf16 output of the int8 path bit-equal to
    the oracle (with bias), per-tensor fp8 with bias and row / column fp8 within the 1e-2 gate, both
    fp8 formats; the kernel each call landed on is checked."""
    print(f"case m={m} n={n} k={k}", flush=True)
    g = torch.Generator().manual_seed(m * 5 + n * 3 + k)
    a, b = _rand_i8(g, m, k), _rand_i8(g, n, k)
    sx = torch.rand(m, 1, generator=g) * 0.05 + 0.01
    sw = torch.rand(n, generator=g) * 0.01 + 0.001
    bias = torch.randn(n, generator=g).to(torch.bfloat16)
    got = C.mm_int8(a.to(DEV), b.to(DEV), sx.to(DEV), sw.to(DEV), bias.to(DEV), 0)
    assert C.last_kernel() == "small64", C.last_kernel()
    want = O.int8_gemm(a, b, sx, sw, bias)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    for fmt, dt in ((0, torch.float8_e4m3fn), (1, torch.float8_e5m2)):
        a8 = (torch.randn(m, k, generator=g) * 1.5).to(dt)
        b8 = (torch.randn(n, k, generator=g) * 1.5).to(dt)
        sa, sb = torch.tensor([0.37]), torch.tensor([0.011])
        out = C.mm_fp8(a8.to(DEV), b8.to(DEV), sa.to(DEV), sb.to(DEV), 0, None, bias.to(DEV))
        assert C.last_kernel() == "small64", C.last_kernel()
        assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa, sb, bias), what=f"small tiles, fmt {fmt}, per tensor + bias")
        sa_r = torch.exp2(torch.rand(m, 1, generator=g) * 6.0 - 3.0)
        sb_r = torch.exp2(torch.rand(n, generator=g) * 6.0 - 3.0)
        out = C.mm_fp8(a8.to(DEV), b8.to(DEV), sa_r.to(DEV), sb_r.to(DEV), 0, None, None)
        assert C.last_kernel() == "small64", C.last_kernel()
        assert_bf16_close(out, O.fp8_gemm_bias(a8, b8, sa_r, sb_r, None), what=f"small tiles, fmt {fmt}, row/column steps")
