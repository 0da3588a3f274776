"""Pins the oracle's fp8 casts (torch's e4m3fn / e5m2 casts, and the C codec)
against tables derived from the OCP format definition with exact rationals."""

import math
import struct

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import w8a8_oracle as O

FMT = {"e4m3fn": (0, torch.float8_e4m3fn), "e5m2": (1, torch.float8_e5m2)}


def _f32(bits: int) -> float:
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def _expected(entry):
    if entry == "nan":
        return math.nan
    if entry in ("inf", "-inf"):
        return float(entry)
    return float.fromhex(entry)


@pytest.mark.parametrize("name", ["e4m3fn", "e5m2"])
def test_decode_table_exhaustive(golden, name):
    table = golden("fp8_codes.json")[f"{name}_decode"]
    fmt, dtype = FMT[name]
    codes = torch.arange(256, dtype=torch.uint8)
    got_torch = codes.view(dtype).float()
    dec = getattr(c_oracle.lib(), f"oracle_{name}_decode")
    for c in range(256):
        want = _expected(table[c])
        gt, gc = got_torch[c].item(), dec(c)
        if math.isnan(want):
            assert math.isnan(gt) and math.isnan(gc), c
        else:
            assert gt == want and gc == want, (c, gt, gc, want)
            # sign of zero
            assert math.copysign(1.0, gt) == math.copysign(1.0, want)


@pytest.mark.parametrize("name", ["e4m3fn", "e5m2"])
def test_cast_rne_ties_subnormals_overflow(golden, name):
    vecs = golden("fp8_codes.json")[f"{name}_cast"]
    fmt, dtype = FMT[name]
    xs = torch.tensor([_f32(b) for b, _ in vecs], dtype=torch.float32)
    want = torch.tensor([c for _, c in vecs], dtype=torch.uint8)
    got = xs.to(dtype).view(torch.uint8)
    enc = getattr(c_oracle.lib(), f"oracle_{name}_encode")
    nan_codes = {0x7F, 0xFF} if name == "e4m3fn" else set(range(0x7D, 0x80)) | set(range(0xFD, 0x100))
    for i, (b, c) in enumerate(vecs):
        gt, gc = int(got[i]), enc(_f32(b))
        if c in nan_codes:
            assert gt in nan_codes and gc in nan_codes, (hex(b), gt, gc, c)
        else:
            assert gt == c and gc == c, (hex(b), _f32(b), gt, gc, c)


def test_rounding_and_overflow_boundaries():
    # e4m3fn: 17->16, 19->20, 21->20, 23->24 (ties to even), 2^-10 -> 0, 464 -> 448, 465 -> NaN
    x = torch.tensor([17.0, 19.0, 21.0, 23.0, 2.0**-10, 464.0, 465.0])
    y = x.to(torch.float8_e4m3fn).float()
    assert y[:6].tolist() == [16.0, 20.0, 20.0, 24.0, 0.0, 448.0]
    assert math.isnan(y[6].item())
    z = torch.tensor([61439.0, 61440.0]).to(torch.float8_e5m2).float()
    assert z[0].item() == 57344.0 and math.isinf(z[1].item())


def test_all_bf16_inputs_c_codec_equals_torch_cast():
    """Every finite bf16 value, three scales, both formats: C encode == torch cast."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    finite = torch.isfinite(x.float())
    for scale in (0.5, 0.0123, 3.0):
        for fmt in (0, 1):
            want, _ = O.fp8_quantize(x, torch.tensor([scale]), fmt)
            got, _ = c_oracle.fp8_quantize(bits, scale, fmt, saturate=False)
            w = want.view(torch.uint8).numpy()
            nanset = (0x7F, 0xFF) if fmt == 0 else tuple(range(0x7D, 0x80)) + tuple(range(0xFD, 0x100))
            w_nan = np.isin(w, nanset)
            g_nan = np.isin(got, nanset)
            f = finite.numpy()
            assert np.array_equal(w_nan[f], g_nan[f])
            ok = f & ~w_nan
            assert np.array_equal(w[ok], got[ok]), (scale, fmt)


def test_saturating_variant_equals_plain_cast_in_range_and_clamps_outside():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(64, 64, generator=g) * 3).to(torch.bfloat16)
    s_ok = O.dynamic_scale(x)
    a, _ = O.fp8_quantize(x, s_ok, 0)
    b, _ = O.fp8_quantize_saturating(x, s_ok, 0)
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8))
    s_small = s_ok / 4
    b, amax = O.fp8_quantize_saturating(x, s_small, 0)
    assert b.float().abs().max().item() == 448.0 and not torch.isnan(b.float()).any()
    assert amax.item() == x.abs().max().item()
