"""FP8 kernel interface adapter: same names, signatures, defaults and scale
semantics as the reference's ``astrai/extension/ops/fp8.py``.

- ``quantize_bf16(x, scale, fmt) -> (x8, amax)``          (ops/fp8.py:125-132)
- ``mm_fp8(a8, b8, sa, sb, out_dtype, out_scale) -> out``   (ops/fp8.py:135-154)
- ``linear_forward_fp8(x, w, bias, sx, sw) -> (out, amax_x, amax_w)``  (:157-166)
- ``linear_backward_fp8(g, x, w, masks, sg, sw, sx, fmt)``  (:169-184)

Scales are quantization *steps* (``x8 = x / scale``); every primitive computes
its own inverse; ``amax`` values are returned, never passed in. The custom ops
``custom::fp8_quantize`` / ``custom::fp8_gemm`` keep the reference's schemas
(ops/fp8.py:55-58,85-93) so ``torch.compile`` traces them the same way.

The reference also registers pure-PyTorch ``cpu`` kernels (ops/fp8.py:78-82,
116-122). Those are its CPU oracle; this backend ships no CPU arithmetic at
all, so the ops raise for CPU tensors instead of computing.
"""

from typing import Optional

import torch
from torch.library import custom_op

from astrai_amd.extension.loader import get_module, is_available

# fmt string -> kernel int (0 = E4M3, 1 = E5M2)
_FMT_TO_INT = {"e4m3": 0, "e5m2": 1}

_MOD: Optional[object] = None


def _mod() -> object:
    global _MOD
    if _MOD is None:
        if not is_available("fp8_mm"):
            raise RuntimeError(
                "HIP kernel 'fp8_mm' is not available. Build with `make -C astrai_amd/csrc`."
            )
        _MOD = get_module("fp8_mm")
    return _MOD


def _no_cpu(op: str):
    raise RuntimeError(
        f"{op}: this backend has no CPU implementation; pass tensors on the MI355X device"
    )


def _fmt_int(fmt: str) -> int:
    try:
        return _FMT_TO_INT[fmt]
    except KeyError:
        raise ValueError(f"unsupported fp8 format {fmt!r} (expected 'e4m3' or 'e5m2')")


@custom_op("custom::fp8_quantize", mutates_args=())
def fp8_quantize(
    x: torch.Tensor, scale: torch.Tensor, fmt: int
) -> tuple[torch.Tensor, torch.Tensor]:
    """BF16 -> FP8 quantize with fused amax; returns ``(x8, amax)``."""
    _no_cpu("custom::fp8_quantize")


@fp8_quantize.register_fake
def _fp8_quantize_fake(x, scale, fmt):
    dtype = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    return (
        torch.empty(x.shape, device=x.device, dtype=dtype),
        torch.empty(1, device=x.device, dtype=torch.float32),
    )


@fp8_quantize.register_kernel("cuda")
def _fp8_quantize_cuda(x, scale, fmt):
    if x.dtype != torch.bfloat16:
        raise TypeError(f"fp8 quantize requires bf16 input, got {x.dtype}")
    return _mod().quantize_bf16(x, scale, int(fmt))


@custom_op("custom::fp8_gemm", mutates_args=())
def fp8_gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    sa: torch.Tensor,
    sb: torch.Tensor,
    out_dtype: int = 0,
    out_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """FP8 GEMM: ``a @ b^T * (sa * sb)`` with FP32 accumulation.

    ``out_dtype``: 0 = BF16 (default), 1 = FP8 E4M3 (requires ``out_scale``).
    """
    _no_cpu("custom::fp8_gemm")


@fp8_gemm.register_fake
def _fp8_gemm_fake(a, b, sa, sb, out_dtype=0, out_scale=None):
    dtype = torch.float8_e4m3fn if out_dtype else torch.bfloat16
    return torch.empty((a.size(0), b.size(0)), device=a.device, dtype=dtype)


@fp8_gemm.register_kernel("cuda")
def _fp8_gemm_cuda(a, b, sa, sb, out_dtype=0, out_scale=None):
    if a.dtype != b.dtype or a.dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
        raise TypeError(
            f"fp8 GEMM requires matching fp8 inputs, got {a.dtype}/{b.dtype}"
        )
    return _mod().mm_fp8(a, b, sa, sb, int(out_dtype), out_scale)


def quantize_bf16(x: torch.Tensor, scale: torch.Tensor, fmt: str = "e4m3"):
    """BF16 -> FP8 quantize with fused amax; returns ``(x8, amax)``.

    ``scale`` is the quantization step (device scalar); ``fmt`` selects E4M3 or
    E5M2. ``amax`` is a fresh 1-element float32 tensor.
    """
    return fp8_quantize(x, scale, _fmt_int(fmt))


def amax_bf16(x: torch.Tensor) -> torch.Tensor:
    """``x.abs().amax()`` as a fresh float32 ``[1]`` tensor from one read of a bf16
    device tensor (what dynamic scaling measures before it quantizes)."""
    if x.dtype != torch.bfloat16:
        raise TypeError(f"amax_bf16 requires a bf16 input, got {x.dtype}")
    return _mod().amax_bf16(x)


def amax_ring_push(hist, idx: int, amax, scale, fmax: float, pow2_margin: float) -> None:
    """Delayed scaling's record-then-refresh on device rings, in place, one launch."""
    _mod().amax_ring_push(hist, idx, amax, scale, fmax, pow2_margin)


def mm_fp8_bias(a, b, sa, sb, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``mm_fp8`` to bf16 with the bias added before the single rounding, the
    epilogue of the fused forward (csrc/kernels/fp8/gemm.cuh:405-435)."""
    return _mod().mm_fp8(a, b, sa, sb, 0, None, bias)


def mm_fp8(
    a: torch.Tensor,
    b: torch.Tensor,
    sa: torch.Tensor,
    sb: torch.Tensor,
    out_dtype: str = "bf16",
    out_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Pre-quantized FP8 GEMM: ``a @ b^T * (sa * sb)``; ``out_dtype`` is
    ``"bf16"`` (default) or ``"e4m3"`` (requires ``out_scale``)."""
    if out_dtype not in ("bf16", "e4m3"):
        raise ValueError(
            f"unsupported out_dtype {out_dtype!r} (expected 'bf16' or 'e4m3')"
        )
    return fp8_gemm(a, b, sa, sb, int(out_dtype == "e4m3"), out_scale)


def linear_forward_fp8(x, w, bias, sx, sw):
    """BF16 linear forward through E4M3; returns ``(out, amax_x, amax_w)``.
    ``bias`` may be ``None``."""
    if not (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16):
        raise TypeError(f"fp8 forward requires bf16 inputs, got {x.dtype}/{w.dtype}")
    if bias is None:
        bias = torch.empty(0, device=x.device, dtype=x.dtype)
    return _mod().linear_forward_fp8(x, w, bias, sx, sw)


def linear_backward_fp8(g, x, w, masks, sg, sw, sx, fmt: str = "e5m2"):
    """FP8 linear backward; returns ``(grad_input, grad_weight, grad_bias, amax_g)``."""
    if not (
        g.dtype == torch.bfloat16
        and x.dtype == torch.bfloat16
        and w.dtype == torch.bfloat16
    ):
        raise TypeError(
            f"fp8 backward requires bf16 inputs, got {g.dtype}/{x.dtype}/{w.dtype}"
        )
    return _mod().linear_backward_fp8(g, x, w, list(masks), sg, sw, sx, _fmt_int(fmt))
