"""Pins the oracle's GEMM / quantize / recipe functions against the reference's
own hand vectors, exact-rational and integer brute force (tests/golden), the
independent C restatement, and identities the mathematics fixes."""

import struct

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import w8a8_oracle as O


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy()


def _bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ---- the reference's hand vectors (tests/extension/test_fp8_mma.py:206-293) ----

def test_reference_kat_mm_fp8(golden):
    k = golden("reference_kats.json")["mm_fp8_cpu"]
    a8 = torch.tensor(k["a8"], dtype=torch.float8_e4m3fn)
    b8 = torch.tensor(k["b8"], dtype=torch.float8_e4m3fn)
    out = O.fp8_gemm(a8, b8, torch.tensor([k["sa"]]), torch.tensor([k["sb"]]))
    assert out.dtype == torch.bfloat16
    assert out.tolist() == k["out_bf16"]


def test_reference_kat_mm_fp8_fp8_out(golden):
    k = golden("reference_kats.json")["mm_fp8_fp8_out_cpu"]
    a8 = torch.tensor(k["a8"], dtype=torch.float8_e4m3fn)
    b8 = torch.tensor(k["b8"], dtype=torch.float8_e4m3fn)
    out = O.fp8_gemm(a8, b8, torch.tensor([k["sa"]]), torch.tensor([k["sb"]]), 1,
                     torch.tensor([k["out_scale"]]))
    assert out.dtype == torch.float8_e4m3fn
    assert out.float().tolist() == k["out_e4m3"]


def test_reference_kat_recipes(golden):
    for r in golden("reference_kats.json")["recipe"]:
        got = O.scale_from_amax(torch.tensor(r["hist"]), r["fmt"], r["margin"])
        assert torch.allclose(got, torch.tensor(r["scale"]))


def test_reference_kat_quantize_scale_half(golden):
    s = golden("reference_kats.json")["quantize_scale"]
    torch.manual_seed(3)
    x = torch.randn(64, 128).to(torch.bfloat16)
    x8, amax = O.fp8_quantize(x, torch.tensor([s]), 0)
    # power-of-two step: x/0.5 is exact, so the codes are the RNE cast of 2x
    assert torch.equal(x8.view(torch.uint8), (x.float() * 2).to(torch.float8_e4m3fn).view(torch.uint8))
    assert amax.item() == x.abs().max().item()
    got, amax_c = c_oracle.fp8_quantize(_bf16_bits(x), s, 0, saturate=False)
    assert np.array_equal(got, _bits(x8)) and amax_c == amax.item()


# ---- fp8 GEMM: exact rationals, C loop, identities ----

def test_fp8_gemm_exact_small(golden):
    for c in golden("fp8_gemm_small.json")["per_tensor"]:
        a8 = torch.tensor(c["a"], dtype=torch.uint8).view(torch.float8_e4m3fn)
        b8 = torch.tensor(c["b"], dtype=torch.uint8).view(torch.float8_e4m3fn)
        exact = torch.tensor(c["exact"], dtype=torch.float64)
        out = O.fp8_gemm(a8, b8, torch.tensor([c["sa"]]), torch.tensor([c["sb"]]))
        want = exact.to(torch.bfloat16)
        # fp32 accumulation error is far below a bf16 ulp except at rounding ties
        torch.testing.assert_close(out.float(), want.float(), rtol=2 ** -7, atol=0)
        cc = c_oracle.fp8_gemm_f32(np.array(c["a"]), np.array(c["b"])) * c["sa"] * c["sb"]
        np.testing.assert_allclose(cc, exact.numpy(), rtol=1e-5)


def test_fp8_gemm_matches_c_loop_and_float64():
    g = torch.Generator().manual_seed(11)
    a = torch.randn(33, 160, generator=g).to(torch.bfloat16)
    b = torch.randn(21, 160, generator=g).to(torch.bfloat16)
    sa, sb = O.dynamic_scale(a), O.dynamic_scale(b)
    a8, _ = O.fp8_quantize(a, sa, 0)
    b8, _ = O.fp8_quantize(b, sb, 0)
    f64 = a8.double() @ b8.double().t() * sa.double() * sb.double()
    got = O.fp8_gemm(a8, b8, sa, sb)
    torch.testing.assert_close(got.double(), f64, rtol=2 ** -7, atol=1e-6)
    c = c_oracle.fp8_gemm_f32(_bits(a8), _bits(b8))
    np.testing.assert_allclose(c * sa.item() * sb.item(), f64.numpy(), rtol=1e-4, atol=1e-4)


def test_fp8_gemm_transposed_operand_or_dropped_scale_would_fail():
    # asymmetric shapes and distinct scales: a@b.T (not a.T@b), both scales applied
    a8 = torch.tensor([[1.0, 2.0, 4.0], [0.5, -1.0, 8.0]]).to(torch.float8_e4m3fn)
    b8 = torch.tensor([[1.0, 1.0, 1.0], [2.0, 0.0, -1.0], [0.0, 3.0, 0.5], [1.0, -2.0, 0.25]]).to(torch.float8_e4m3fn)
    out = O.fp8_gemm(a8, b8, torch.tensor([2.0]), torch.tensor([0.25]))
    want = torch.tensor([[7.0, -2.0, 8.0, -2.0], [7.5, -7.0, 1.0, 4.5]]) * 0.5
    assert out.shape == (2, 4) and torch.equal(out.float(), want)


def test_bias_epilogue_single_rounding():
    a8 = torch.tensor([[1.0, 2.0]]).to(torch.float8_e4m3fn)
    b8 = torch.tensor([[3.0, 4.0]]).to(torch.float8_e4m3fn)
    # 11 * 1.0009765625 = 11.0107..., + 0.03 -> one rounding of the fp32 sum
    sa, sb = torch.tensor([1.0009765625]), torch.tensor([1.0])
    bias = torch.tensor([0.03125]).to(torch.bfloat16)
    got = O.fp8_gemm_bias(a8, b8, sa, sb, bias)
    assert got.item() == torch.tensor(11.0 * 1.0009765625 + 0.03125).to(torch.bfloat16).item()
    assert torch.equal(O.fp8_gemm_bias(a8, b8, sa, sb, None), O.fp8_gemm(a8, b8, sa, sb))


def test_linear_forward_fp8_formula_of_reference_test():
    # tests/extension/test_fp8_mma.py:88-116 expected-value formula, m,n,k = 19,13,37, seed 7
    torch.manual_seed(7)
    m, n, k = 19, 13, 37
    x = torch.randn(m, k).to(torch.bfloat16)
    w = torch.randn(n, k).to(torch.bfloat16)
    bias = torch.randn(n).to(torch.bfloat16)
    sx = (x.abs().amax().float() / 448.0).clamp_min(1e-12)
    sw = (w.abs().amax().float() / 448.0).clamp_min(1e-12)
    out, ax, aw = O.linear_forward_fp8(x, w, bias, sx, sw)
    qx = (x.float() / sx).to(torch.float8_e4m3fn).float()
    qw = (w.float() / sw).to(torch.float8_e4m3fn).float()
    want = (qx @ qw.t() * sx * sw + bias).to(torch.bfloat16)
    torch.testing.assert_close(out, want, atol=0.125, rtol=0.01)
    assert ax.item() == x.abs().max().item() and aw.item() == w.abs().max().item()


# ---- int8 ----

def test_int8_gemm_integer_brute_force(golden):
    for c in golden("int8_small.json")["gemm"]:
        a = torch.tensor(c["a"], dtype=torch.int8)
        b = torch.tensor(c["b"], dtype=torch.int8)
        want = torch.tensor(c["acc"], dtype=torch.int32)
        assert torch.equal(O.int8_acc(a, b), want)
        assert np.array_equal(c_oracle.int8_gemm_i32(a.numpy(), b.numpy()), want.numpy())


def test_int8_quantize_rows_exact(golden):
    for c in golden("int8_small.json")["quantize_rows"]:
        x = torch.tensor([c["x"]], dtype=torch.float32).to(torch.bfloat16)
        assert torch.equal(x.float(), torch.tensor([c["x"]]))  # fixture values are bf16-exact
        q, s = O.int8_quantize_rows(x)
        assert struct.unpack("<I", struct.pack("<f", s.item()))[0] == c["scale_bits"]
        assert q[0].tolist() == c["q"]
        qc, sc = c_oracle.int8_quantize_rows(_bf16_bits(x))
        assert qc[0].tolist() == c["q"] and sc[0] == s.item()


def test_int8_quantize_rows_c_equals_torch_random():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(37, 200, generator=g).to(torch.bfloat16)
    q, s = O.int8_quantize_rows(x)
    qc, sc = c_oracle.int8_quantize_rows(_bf16_bits(x))
    assert np.array_equal(q.numpy(), qc) and np.array_equal(s.reshape(-1).numpy(), sc)
    assert q.abs().max().item() == 127  # symmetric: the row max maps to +-127


def test_int8_gemm_epilogue_scales_rows_and_columns():
    xq = torch.tensor([[1, 2], [3, 4], [-5, 6]], dtype=torch.int8)
    wq = torch.tensor([[1, 0], [0, 1]], dtype=torch.int8)
    sx = torch.tensor([[1.0], [0.5], [2.0]])
    sw = torch.tensor([1.0, 4.0])
    out = O.int8_gemm(xq, wq, sx, sw)
    assert out.float().tolist() == [[1.0, 8.0], [1.5, 8.0], [-10.0, 48.0]]
    bias = torch.tensor([0.5, -1.0]).to(torch.bfloat16)
    assert O.int8_gemm(xq, wq, sx, sw, bias).float().tolist() == [[1.5, 7.0], [2.0, 7.0], [-9.5, 47.0]]


def test_int8_config0_fp32_matmul_would_not_be_exact_but_int_is():
    x, w, _ = O.make_inputs(0, 16, 64, 2048)
    xq, _ = O.int8_quantize_rows(x)
    wq, _ = O.int8_quantize_rows(w)
    acc = O.int8_acc(xq, wq)
    assert np.array_equal(acc.numpy(), c_oracle.int8_gemm_i32(xq.numpy(), wq.numpy()))
    assert torch.equal(acc, (xq.double() @ wq.double().t()).to(torch.int32))


def test_int8_acc_every_route_equals_int32_matmul_and_c_loop():
    """The accumulator's three routes (int32 matmul, exact float64 matmul, and the opt-in
    library int8 routine with its sampled self-check) on ragged shapes, a decode shape, a
    multi-tile shape and worst-case magnitudes (every product +-127^2, K = 4096: |acc| = 66 M,
    no wrap) against the int32 tensor matmul and the C triple loop."""
    g = torch.Generator().manual_seed(11)
    for m, n, k in ((1, 5, 1), (4, 3, 1), (3, 5, 7), (2, 3, 15), (5, 4, 16), (17, 9, 33), (1, 300, 4096), (130, 257, 1000), (64, 96, 4096)):
        a = torch.randint(-127, 128, (m, k), dtype=torch.int8, generator=g)
        b = torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g)
        want = O.int8_acc_int32_matmul(a, b)
        for fast in (False, True):
            got = O.int8_acc(a, b, fast=fast)
            assert got.dtype == torch.int32 and torch.equal(got, want), (m, n, k, fast)
        if m * n * k <= 4_000_000:
            assert np.array_equal(want.numpy(), c_oracle.int8_gemm_i32(a.numpy(), b.numpy())), (m, n, k)
    a = torch.full((5, 4096), 127, dtype=torch.int8)
    a[1::2] = -127
    b = torch.full((7, 4096), -127, dtype=torch.int8)
    b[::3] = 127
    want = O.int8_acc_int32_matmul(a, b)
    assert want.abs().max().item() == 127 * 127 * 4096
    assert torch.equal(O.int8_acc(a, b), want) and torch.equal(O.int8_acc(a, b, fast=True), want)
    # the float64 route (products too large for the int32 matmul's time) on worst-case magnitudes
    a = torch.full((300, 4096), 127, dtype=torch.int8)
    a[1::2] = -127
    b = torch.full((260, 4096), -127, dtype=torch.int8)
    b[::3] = 127
    assert 300 * 260 * 4096 > (1 << 24)
    assert torch.equal(O.int8_acc(a, b), O.int8_acc_int32_matmul(a, b))
    # a strided view takes the same routes
    assert torch.equal(O.int8_acc(a[:, ::2], b[:, ::2]), O.int8_acc_int32_matmul(a[:, ::2], b[:, ::2]))


def test_int8_acc_fast_route_raises_on_a_wrong_library_result(monkeypatch):
    a = torch.randint(-127, 128, (8, 64), dtype=torch.int8)
    b = torch.randint(-127, 128, (8, 64), dtype=torch.int8)
    real = torch._int_mm
    monkeypatch.setattr(torch, "_int_mm", lambda x, y: real(x, y) + 1)
    with pytest.raises(RuntimeError, match="disagrees"):
        O.int8_acc(a, b, fast=True)


def test_block128_reduces_to_per_tensor_when_scales_equal():
    g = torch.Generator().manual_seed(4)
    a = torch.randn(9, 384, generator=g).to(torch.bfloat16)
    b = torch.randn(200, 384, generator=g).to(torch.bfloat16)
    s = torch.tensor([0.03125])
    a8, _ = O.fp8_quantize(a, s, 0)
    b8, _ = O.fp8_quantize(b, s, 0)
    sa = torch.full((9, 3), 0.03125)
    sb = torch.full((2, 3), 0.03125)
    got = O.fp8_gemm_blockscaled(a8, b8, sa, sb)
    want = O.fp8_gemm(a8, b8, s, s)
    # power-of-two scales commute exactly with the fp32 sums; only the sum order differs
    torch.testing.assert_close(got.float(), want.float(), rtol=2 ** -7, atol=1e-6)


def test_block128_quantizers_scale_layout_and_range():
    x, w, _ = O.make_inputs(3, 5, 200, 256, outlier_p=0.01)
    x8, sa = O.fp8_quantize_act_block128(x)
    w8, sb = O.fp8_quantize_weight_block128(w)
    assert sa.shape == (5, 2) and sb.shape == (2, 2)
    assert torch.equal(sa[:, 1], x[:, 128:].float().abs().amax(dim=1) / 448.0)
    assert sb[1, 0].item() == (w[128:, :128].float().abs().max() / 448.0).item()
    assert x8.float().abs().max().item() == 448.0 and w8.float().abs().max().item() == 448.0
    # dequantized product close to the bf16 product
    ref = x.float() @ w.float().t()
    got = O.fp8_gemm_blockscaled(x8, w8, sa, sb).float()
    assert ((got - ref).abs().max() / ref.abs().max()).item() < 0.05


def test_dynamic_linear_double_rounding_order():
    # bias is added after the bf16 rounding (astrai/extension/fp8.py:296-298)
    x, w, b = O.make_inputs(1, 4, 8, 32, w_std=1.0, bias=True)
    out = O.fp8_linear_dynamic(x, w, b)
    nb = O.fp8_linear_dynamic(x, w, None)
    assert torch.equal(out, nb + b)
