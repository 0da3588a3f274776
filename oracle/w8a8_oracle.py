"""CPU restatement of the reference's quantized-linear arithmetic (pure PyTorch).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; never by the product package.

Every function cites the reference lines it follows (paths relative to the
reference checkout). Functions for int8 per-token x per-channel and 128-block
fp8 scaling have no counterpart in the reference (it is per-tensor fp8 only);
they extend its CPU kernels with the same conventions: a scale is the
*quantization step* (``q = x / scale``; dequantization multiplies by it),
accumulation is exact int32 / fp32, scales enter by broadcasting, and the result
is rounded once to bf16.

Pinning (see tests/test_oracle_*.py):
  * e4m3fn / e5m2 casts  -> exhaustive 256-code decode tables and nearest/tie
    vectors derived from the OCP format definition with exact rationals
    (tests/golden/fp8_codes.json), plus the independent C restatement in
    oracle/w8a8_oracle.c.
  * fp8_quantize / fp8_gemm -> the reference's own hand vectors
    (tests/extension/test_fp8_mma.py:262-293) and exact-rational brute force.
  * int8 ops -> pure-Python integer triple loops (tests/golden/int8_small.json)
    and the C triple loop.
  * block-scaled GEMM -> exact-rational brute force on small shapes and the
    reduction to the per-tensor GEMM when all block scales are equal.
  * recipes -> the reference's closed-form numbers (test_fp8_mma.py:206-222).
"""

from __future__ import annotations

import torch

FP8_MAX = {"e4m3": 448.0, "e5m2": 57344.0}  # astrai/extension/fp8.py:43
INT8_MAX = 127.0
BLOCK = 128


def fmt_dtype(fmt: int) -> torch.dtype:
    """0 = E4M3 (OCP e4m3fn), 1 = E5M2. astrai/extension/ops/fp8.py:24-25,51-52."""
    return torch.float8_e5m2 if fmt else torch.float8_e4m3fn


# ---------------------------------------------------------------------------
# fp8 per-tensor: the two CPU kernels of the reference
# ---------------------------------------------------------------------------


def fp8_quantize(x: torch.Tensor, scale: torch.Tensor, fmt: int):
    """``custom::fp8_quantize`` CPU kernel. astrai/extension/ops/fp8.py:78-82.

    ``x8 = (x.float() / scale).to(fp8)``; amax over the raw values, clamped
    below at 1e-12 (CPU path only; the device kernel returns the bare max,
    csrc/kernels/fp8/mm.cu:115).
    """
    x8 = (x.float() / scale).to(fmt_dtype(fmt))
    amax = x.abs().amax().float().reshape(1).clamp_min(1e-12)
    return x8, amax


def fp8_quantize_saturating(x: torch.Tensor, scale: torch.Tensor, fmt: int):
    """Device-kernel variant: saturate to the format's finite max instead of NaN.

    csrc/kernels/fp8/gemm.cuh:35-42,128-146 convert with ``__NV_SATFINITE``;
    the plain torch cast yields NaN above the rounding boundary (e4m3fn) or
    inf (e5m2). Identical to :func:`fp8_quantize` whenever ``scale >= amax/max``.
    amax is the bare max of |x| (zero-initialised atomic max, mm.cu:115).
    """
    lim = FP8_MAX["e5m2" if fmt else "e4m3"]
    q = (x.float() / scale).clamp(-lim, lim)
    x8 = q.to(fmt_dtype(fmt))
    amax = x.abs().amax().float().reshape(1)
    return x8, amax


def fp8_gemm(a, b, sa, sb, out_dtype: int = 0, out_scale=None):
    """``custom::fp8_gemm`` CPU kernel. astrai/extension/ops/fp8.py:116-122.

    ``acc = a.float() @ b.float().t() * sa * sb``; bf16 out, or e4m3fn out after
    multiplying by ``out_scale`` (1.0 when absent).
    """
    acc = a.float() @ b.float().t() * sa * sb
    if out_dtype:
        os_ = 1.0 if out_scale is None else out_scale
        return (acc * os_).to(torch.float8_e4m3fn)
    return acc.to(torch.bfloat16)


def fp8_gemm_bias(a, b, sa, sb, bias=None):
    """Pre-quantized GEMM with the fused-kernel epilogue: scale, add bias in
    fp32, round once to bf16. csrc/kernels/fp8/gemm.cuh:405-435."""
    acc = a.float() @ b.float().t() * sa * sb
    if bias is not None and bias.numel():
        acc = acc + bias.float()
    return acc.to(torch.bfloat16)


def linear_forward_fp8(x, w, bias, sx, sw):
    """Fused bf16 -> e4m3 -> GEMM -> bf16 linear forward; returns
    ``(out, amax_x, amax_w)``. csrc/kernels/fp8/mm.cu:186-234 (contract),
    gemm.cuh:405-435 (epilogue), tests/extension/test_fp8_mma.py:104-116
    (expected-value formula used by the reference's own test)."""
    k = w.size(1)
    x2 = x.reshape(-1, k)
    x8, _ = fp8_quantize_saturating(x2, sx, 0)
    w8, _ = fp8_quantize_saturating(w, sw, 0)
    out = fp8_gemm_bias(x8, w8, sx, sw, bias)
    amax_x = x.abs().amax().float().reshape(1)
    amax_w = w.abs().amax().float().reshape(1)
    return out.reshape(*x.shape[:-1], w.size(0)), amax_x, amax_w


def scale_from_amax(amax: torch.Tensor, fmt: str, margin: int = 0) -> torch.Tensor:
    """``scale = (max(hist) / FP8_MAX[fmt]) / 2^margin`` clamped at 1e-12.
    astrai/extension/fp8.py:87-89,103-105."""
    return ((amax.max() / FP8_MAX[fmt]) / (2**margin)).clamp_min(1e-12)


def dynamic_scale(t: torch.Tensor, fmt: str = "e4m3", margin: int = 0) -> torch.Tensor:
    """astrai/extension/fp8.py:270-272."""
    amax = t.abs().amax().to(torch.float32).clamp_min(1e-12)
    return scale_from_amax(amax, fmt, margin)


def fp8_linear_dynamic(x, w, bias=None):
    """DynamicScaling forward: measure, quantize both, GEMM to bf16, add bias
    *after* the bf16 rounding. astrai/extension/fp8.py:289-299."""
    x2 = x.reshape(-1, w.size(1))
    sx = dynamic_scale(x2)
    sw = dynamic_scale(w)
    x8, _ = fp8_quantize(x2, sx, 0)
    w8, _ = fp8_quantize(w, sw, 0)
    out = fp8_gemm(x8, w8, sx, sw).reshape(*x.shape[:-1], w.size(0))
    if bias is not None and bias.numel():
        out = out + bias
    return out


# ---------------------------------------------------------------------------
# int8 per-token x per-channel (extension of the same conventions)
# ---------------------------------------------------------------------------


def int8_quantize_rows(x: torch.Tensor):
    """Symmetric per-row int8: ``s[r] = max|x[r,:]| / 127`` (amax clamped at
    1e-12 like astrai/extension/fp8.py:271), ``q = clamp(rne(x / s), +-127)``.
    Used per token for activations and per output channel for weights.
    Returns ``(q int8 [R,K], s fp32 [R,1])``."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    s = amax / INT8_MAX
    q = torch.round(xf / s).clamp(-INT8_MAX, INT8_MAX).to(torch.int8)
    return q, s


def int8_acc_int32_matmul(xq: torch.Tensor, wq: torch.Tensor) -> torch.Tensor:
    """Exact int32 accumulator ``xq @ wq^T`` as a plain int32 tensor matmul."""
    return xq.to(torch.int32) @ wq.to(torch.int32).t()


def int8_acc(xq: torch.Tensor, wq: torch.Tensor, fast: bool = False) -> torch.Tensor:
    """Exact int32 accumulator ``xq @ wq^T``. fp32 matmul of int8 values is not exact once
    K*127^2 >= 2^24, so the default is arithmetic that is exact by construction: the int32
    tensor matmul for small products and, for large ones, a float64 matmul -- every partial
    sum is an integer of magnitude <= K*127^2 < 2^53, so each double addition is exact in
    any order the BLAS chooses (0.8 s at 4096^3 on eight cores).

    ``fast=True`` (timing legs only) takes PyTorch's int8 x int8 -> int32 CPU routine,
    ``torch._int_mm``: ~15x faster, private, and known to return garbage for K = 1; every
    such call re-computes a random subset of rows with the int32 matmul and raises on a
    mismatch, and short contractions never reach it."""
    if not (xq.numel() and wq.numel()):
        return int8_acc_int32_matmul(xq, wq)
    m, k, n = xq.size(0), xq.size(-1), wq.size(0)
    if fast and xq.dtype == torch.int8 and wq.dtype == torch.int8 and k >= 16:
        out = torch._int_mm(xq.contiguous(), wq.contiguous().t())
        rows = torch.randint(0, m, (min(m, 4),))
        if not torch.equal(out[rows], int8_acc_int32_matmul(xq[rows], wq)):
            raise RuntimeError(f"torch._int_mm disagrees with the int32 matmul at {m}x{n}x{k}")
        return out
    if m * n * k <= (1 << 24):
        return int8_acc_int32_matmul(xq, wq)
    assert k * 127 * 127 < (1 << 53)
    return (xq.double() @ wq.double().t()).to(torch.int32)


def int8_gemm(xq, wq, sx, sw, bias=None, fast: bool = False):
    """``bf16(acc * sx[m] * sw[n] (+ bias[n]))`` with the broadcast-scale form of
    astrai/extension/ops/fp8.py:118 and the single-rounding epilogue of
    csrc/kernels/fp8/gemm.cuh:405-435. ``fast``: see :func:`int8_acc` (timing legs)."""
    acc = int8_acc(xq, wq, fast=fast).float() * sx.reshape(-1, 1).float() * sw.reshape(1, -1).float()
    if bias is not None and bias.numel():
        acc = acc + bias.float()
    return acc.to(torch.bfloat16)


def int8_linear(x, wq, sw, bias=None, fast: bool = False):
    """W8A8 linear: per-token quantize ``x`` then :func:`int8_gemm`."""
    k = wq.size(1)
    xq, sx = int8_quantize_rows(x.reshape(-1, k))
    out = int8_gemm(xq, wq, sx, sw, bias, fast=fast)
    return out.reshape(*x.shape[:-1], wq.size(0))


# ---------------------------------------------------------------------------
# fp8 with 128-block scales (extension of the same conventions)
# ---------------------------------------------------------------------------


def _ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def fp8_quantize_act_block128(x: torch.Tensor):
    """Activation scales per 1x128 K-group: ``sa[m,kb] = max|x[m,128kb:..]|/448``.
    K must be a multiple of 128. Returns ``(x8 e4m3fn [M,K], sa fp32 [M,K/128])``."""
    m, k = x.shape
    assert k % BLOCK == 0
    xf = x.float().reshape(m, k // BLOCK, BLOCK)
    amax = xf.abs().amax(dim=-1).clamp_min(1e-12)
    sa = amax / FP8_MAX["e4m3"]
    x8 = (xf / sa[..., None]).reshape(m, k).to(torch.float8_e4m3fn)
    return x8, sa


def fp8_quantize_weight_block128(w: torch.Tensor):
    """Weight scales per 128x128 block: ``sb[nb,kb] = max|w[blk]|/448``. N may be
    ragged (last block short). Returns ``(w8 [N,K], sb fp32 [ceil(N/128),K/128])``."""
    n, k = w.shape
    assert k % BLOCK == 0
    nb, kb = _ceil_div(n, BLOCK), k // BLOCK
    wf = w.float()
    pad = nb * BLOCK - n
    wp = torch.nn.functional.pad(wf, (0, 0, 0, pad)) if pad else wf
    blk = wp.reshape(nb, BLOCK, kb, BLOCK)
    amax = blk.abs().amax(dim=(1, 3)).clamp_min(1e-12)
    sb = amax / FP8_MAX["e4m3"]
    w8 = (blk / sb[:, None, :, None]).reshape(nb * BLOCK, k)[:n].to(torch.float8_e4m3fn)
    return w8, sb


def fp8_gemm_blockscaled(a8, b8, sa, sb, bias=None):
    """``out[m,n] = bf16( sum_kb (a8[m,kb] . b8[n,kb]) * sa[m,kb] * sb[n//128,kb] )``
    with fp32 accumulation over K-blocks, following the scale-after-dot order of
    astrai/extension/ops/fp8.py:118 applied per 128-wide K-block."""
    m, k = a8.shape
    n = b8.shape[0]
    kb = k // BLOCK
    af = a8.float().reshape(m, kb, BLOCK)
    bf = b8.float().reshape(n, kb, BLOCK)
    sb_rows = sb.repeat_interleave(BLOCK, dim=0)[:n]  # [N, KB]
    acc = torch.zeros(m, n, dtype=torch.float32)
    for i in range(kb):
        part = af[:, i, :] @ bf[:, i, :].t()
        acc += part * sa[:, i].reshape(-1, 1) * sb_rows[:, i].reshape(1, -1)
    if bias is not None and bias.numel():
        acc = acc + bias.float()
    return acc.to(torch.bfloat16)


def add_rmsnorm_quantize_int8(x, weight, eps, res=None):
    """Residual add, RMSNorm and per-token int8 as the decoder computes them one
    after the other: ``t = x + res`` in bf16 (astrai/model/components/
    decoder_block.py:59-70), ``y = F.rms_norm(t, (K,), weight, eps)``
    (components/norm.py:7-15), then :func:`int8_quantize_rows`. Returns
    ``(xq, s, t, y)``."""
    t = x if res is None else x + res
    y = torch.nn.functional.rms_norm(t, (t.size(-1),), weight, eps)
    xq, s = int8_quantize_rows(y.reshape(-1, y.size(-1)))
    return xq, s, t, y


def silu_mul_quantize_int8(gate, up):
    """``h = up * F.silu(gate)`` in bf16 (astrai/model/components/mlp.py:41), then
    :func:`int8_quantize_rows`. Returns ``(hq, s, h)``."""
    h = up * torch.nn.functional.silu(gate)
    hq, s = int8_quantize_rows(h.reshape(-1, h.size(-1)))
    return hq, s, h


# ---------------------------------------------------------------------------
# Seeded workload generators shared by tests and bench (activation, weight,
# bias, outlier mask drawn in that order from one CPU generator)
# ---------------------------------------------------------------------------


def make_inputs(seed: int, m: int, n: int, k: int, x_std=1.0, w_std=0.02,
                bias: bool = False, outlier_p: float = 0.0, outlier_mul: float = 20.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, k, generator=g) * x_std).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g) * w_std
    b = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16) if bias else None
    if outlier_p > 0:
        mask = torch.rand(n, k, generator=g) < outlier_p
        w = torch.where(mask, w * outlier_mul, w)
    return x, w.to(torch.bfloat16), b
