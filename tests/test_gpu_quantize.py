"""Quantize kernels vs the oracle, bit-exact on codes (HIP path through the C ABI)."""

import numpy as np
import pytest
import torch

from oracle import w8a8_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _codes(t):
    return t.cpu().contiguous().view(torch.uint8)


@pytest.fixture(scope="module")
def C():
    from astrai_amd.extension import _cabi
    assert _cabi.load() is not None, _cabi.load_error()
    return _cabi


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("scale", [0.5, 0.0123, 3.0, 1e-3])
def test_fp8_quantize_every_bf16_value(C, fmt, scale):
    """All 65536 bf16 bit patterns: codes equal the saturating oracle wherever the
    input is finite (RNE, subnormals, ties, saturation at the finite max)."""
    print(f"case fmt={fmt} scale={scale}", flush=True)
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    finite = torch.isfinite(x.float())
    x = torch.where(finite, x, torch.zeros_like(x))
    s = torch.tensor([scale])
    want, want_amax = O.fp8_quantize_saturating(x, s, fmt)
    got, amax = C.quantize_bf16(x.to(DEV), s.to(DEV), fmt)
    assert got.dtype == want.dtype and got.shape == x.shape
    assert torch.equal(_codes(got), _codes(want))
    assert amax.shape == (1,) and amax.item() == want_amax.item()


@pytest.mark.parametrize("fmt", [0, 1])
def test_fp8_quantize_every_bf16_value_many_steps(C, fmt):
    """The quantizer forms its quotients from a reciprocal, an exact remainder and a correction,
    and falls back to the IEEE division only near a rounding point of the conversion: all 65536
    bf16 patterns -- infinities (saturate) and NaNs (stay NaN) included -- under 60 steps: random
    ones, powers of two (every quotient exact, ties everywhere), steps whose reciprocal rounds
    badly (mantissa all ones, just above a power of two), tiny and huge ones (the division path
    throughout), the 1e-12 floor of the scaling policy."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    nan = torch.isnan(x.float())
    g = torch.Generator().manual_seed(77 + fmt)
    steps = torch.exp2(torch.rand(40, generator=g) * 30.0 - 20.0).tolist()
    ones = np.array([0x3fffffff, 0x3f800001, 0x3effffff, 0x40000001, 0x3a7fffff], dtype=np.uint32).view(np.float32)
    steps += [1.0, 0.25, 2.0 ** -9, 64.0, 448.0, 1.0 / 448.0, 57344.0, 1e-12, 2.0 ** -70, 2.0 ** 70,
              2.0 ** -61, 2.0 ** 61, 3.0, 0.1, 7.0 / 448.0] + [float(v) for v in ones]
    xd = x.to(DEV)
    for step in steps:
        s = torch.tensor([step], dtype=torch.float32)
        want, _ = O.fp8_quantize_saturating(torch.where(nan, torch.zeros_like(x), x), s, fmt)
        got, _ = C.quantize_bf16(xd, s.to(DEV), fmt)
        gc, wc = _codes(got), _codes(want)
        bad = (gc != wc) & ~nan
        assert not bad.any(), (f"step {step!r} fmt {fmt}: {int(bad.sum())} codes differ, first at bf16 pattern "
                               f"{int(bad.nonzero()[0])}: got {int(gc[bad][0])} want {int(wc[bad][0])}")
        assert torch.isnan(got.cpu().float()[nan]).all(), f"step {step!r}: a NaN became a number"


def test_fp8_quantize_reference_vector_scale_half(C, golden):
    # tests/extension/test_fp8_mma.py:65-77
    torch.manual_seed(3)
    x = torch.randn(64, 128).to(torch.bfloat16)
    scale = torch.tensor([golden("reference_kats.json")["quantize_scale"]])
    from astrai_amd.extension.ops.fp8 import quantize_bf16
    x8, amax = quantize_bf16(x.to(DEV), scale.to(DEV), "e4m3")
    assert x8.dtype == torch.float8_e4m3fn and x8.shape == x.shape and amax.shape == (1,)
    torch.testing.assert_close(amax.cpu(), x.abs().amax().float().reshape(1))
    ref = (x.float() / 0.5).to(torch.float8_e4m3fn)
    assert torch.equal(_codes(x8), _codes(ref))


@pytest.mark.parametrize("shape", [(1,), (7,), (8,), (3, 5), (257, 33), (0, 16), (4096, 4096)])
def test_fp8_quantize_shapes_tails_and_amax(C, shape):
    print(f"case shape={shape}", flush=True)
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 2).to(torch.bfloat16)
    s = O.dynamic_scale(x) if x.numel() else torch.tensor(1.0)
    s = s.reshape(1)
    got, amax = C.quantize_bf16(x.to(DEV), s.to(DEV), 0)
    assert got.shape == x.shape and got.dtype == torch.float8_e4m3fn
    if x.numel() == 0:  # nothing launched; amax keeps its zero initialisation
        assert amax.item() == 0.0
        return
    want, _ = O.fp8_quantize(x, s, 0)
    assert torch.equal(_codes(got), _codes(want))
    assert amax.item() == x.abs().max().item()


def test_fp8_quantize_noncontiguous_input(C):
    x = torch.randn(64, 96).to(torch.bfloat16)
    xt = x.to(DEV).t()
    s = torch.tensor([0.25])
    got, _ = C.quantize_bf16(xt, s.to(DEV), 0)
    want, _ = O.fp8_quantize(x.t(), s, 0)
    assert got.shape == (96, 64) and torch.equal(_codes(got), _codes(want))


@pytest.mark.parametrize("fmt", [0, 1])
@pytest.mark.parametrize("shape", [(1, 1), (1, 33), (33, 1), (17, 9), (128, 64), (130, 72), (16, 8),
                                   (48, 20), (129, 65), (256, 7), (19, 128), (1000, 520), (0, 8),
                                   (2048, 4096),
                                   (6016, 5896)])   # 47 x 47 tiles: more than one tile per workgroup
def test_fp8_quantize_transposed_codes(C, shape, fmt):
    """One pass gives the codes of x and of x.t().contiguous() (the copies
    csrc/kernels/fp8/mm.cu:298-311 quantizes) and the amax, bit-exact, for
    aligned, ragged and single-row/column matrices."""
    print(f"case shape={shape} fmt={fmt}", flush=True)
    g = torch.Generator().manual_seed(7 + shape[0] * 31 + shape[1])
    x = (torch.randn(*shape, generator=g) * 3).to(torch.bfloat16)
    s = torch.tensor([0.037 if fmt == 0 else 0.0011])
    x8, x8t, amax = C.quantize_transpose_bf16(x.to(DEV), s.to(DEV), fmt, want_rowmajor=True,
                                              want_amax=True)
    assert x8.shape == shape and x8t.shape == (shape[1], shape[0])
    if x.numel() == 0:
        assert amax.item() == 0.0
        return
    want, _ = O.fp8_quantize_saturating(x, s, fmt)
    assert x8.dtype == want.dtype and x8t.dtype == want.dtype
    assert torch.equal(_codes(x8), _codes(want))
    assert torch.equal(_codes(x8t), _codes(want).t().contiguous())
    assert amax.item() == x.abs().max().item()
    none8, only_t, zero = C.quantize_transpose_bf16(x.to(DEV), s.to(DEV), fmt)
    assert none8 is None and zero is None
    assert torch.equal(_codes(only_t), _codes(x8t))


@pytest.mark.parametrize("rows,k", [(1, 8), (3, 24), (16, 2048), (5, 33), (2, 9000), (7, 16384), (64, 4096), (0, 32),
                                    # long blocks: one wave per row up to K = 4096
                                    (16384, 2048), (513, 4096), (1000, 264), (4099, 8), (600, 1032), (700, 4104),
                                    (512, 36)])
def test_int8_rows_bit_exact(C, rows, k):
    print(f"case rows={rows} k={k}", flush=True)
    g = torch.Generator().manual_seed(rows * 31 + k)
    x = torch.randn(rows, k, generator=g).to(torch.bfloat16)
    if rows > 1:
        x[1].zero_()  # all-zero row: step = 1e-12/127, codes 0
    got_q, got_s = C.quantize_int8_rows(x.to(DEV))
    want_q, want_s = O.int8_quantize_rows(x)
    assert got_q.shape == (rows, k) and got_s.shape == (rows, 1)
    assert torch.equal(got_s.cpu(), want_s)
    assert torch.equal(got_q.cpu(), want_q)


def test_int8_rows_golden_ties(C, golden):
    for c in golden("int8_small.json")["quantize_rows"]:
        x = torch.tensor([c["x"]], dtype=torch.float32).to(torch.bfloat16)
        q, s = C.quantize_int8_rows(x.to(DEV))
        assert q.cpu()[0].tolist() == c["q"]
        assert s.cpu().view(torch.int32).item() == c["scale_bits"]


def test_int8_rows_3d_input_flattens_tokens(C):
    x = torch.randn(2, 5, 64).to(torch.bfloat16)
    q, s = C.quantize_int8_rows(x.to(DEV))
    wq, ws = O.int8_quantize_rows(x.reshape(-1, 64))
    assert q.shape == (10, 64) and torch.equal(q.cpu(), wq) and torch.equal(s.cpu(), ws)


@pytest.mark.parametrize("m,k", [(1, 128), (5, 256), (130, 1024)])
def test_block128_act_quantize(C, m, k):
    x, _, _ = O.make_inputs(3, m, 8, k)
    x8, sa = C.quantize_fp8_block128_act(x.to(DEV))
    w8, ws = O.fp8_quantize_act_block128(x)
    assert torch.equal(sa.cpu(), ws) and torch.equal(_codes(x8), _codes(w8))


@pytest.mark.parametrize("n,k", [(128, 128), (200, 256), (1, 128), (257, 384)])
def test_block128_weight_quantize(C, n, k):
    _, w, _ = O.make_inputs(3, 4, n, k, outlier_p=0.01)
    w8, sb = C.quantize_fp8_block128_weight(w.to(DEV))
    r8, rs = O.fp8_quantize_weight_block128(w)
    assert sb.shape == rs.shape and torch.equal(sb.cpu(), rs)
    assert torch.equal(_codes(w8), _codes(r8))


def test_quantizer_random_shape_sweep(C):
    """Seeded random shapes through the three quantizers (the checks of the parametrized tests
    above): transposed fp8 codes, per-row int8, 128-block fp8."""
    g = torch.Generator().manual_seed(606)
    r = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for i in range(12):
        test_fp8_quantize_transposed_codes(C, (r(1, 700), r(1, 700)), i % 2)
    for i in range(12):
        test_int8_rows_bit_exact(C, r(1, 80), r(1, 12000))
    for i in range(6):
        test_block128_act_quantize(C, r(1, 400), 128 * r(1, 12))
        test_block128_weight_quantize(C, r(1, 600), 128 * r(1, 8))
