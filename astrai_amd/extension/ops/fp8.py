"""fp8 primitives of the MI355X backend, behind the call surface AstrAI's policy
layer uses (reference: ``astrai/extension/ops/fp8.py``).

What the reference exposes and where (all in its ``ops/fp8.py``):

===========================  ============================================  =========
callable                     returns                                       lines
===========================  ============================================  =========
``quantize_bf16``            ``(codes, amax)``                             125-132
``mm_fp8``                   ``a8 @ b8.T * sa * sb`` (bf16 or e4m3)        135-154
``linear_forward_fp8``       ``(out, amax_x, amax_w)``                     157-166
``linear_backward_fp8``      ``(grad_x, grad_w, grad_bias, amax_grad)``    169-184
``custom::fp8_quantize``     dispatcher op behind ``quantize_bf16``        55-58
``custom::fp8_gemm``         dispatcher op behind ``mm_fp8``               85-93
===========================  ============================================  =========

Conventions kept from there: a scale is the quantization step (codes are
``x / scale``, results are multiplied by it), nobody passes reciprocals, an
amax is handed back as a fresh one-element fp32 tensor. Format names are
``"e4m3"`` / ``"e5m2"``, output names ``"bf16"`` / ``"e4m3"``; their position in
the tuples below is the integer the kernels take.

Like the reference, the two dispatcher ops carry three registrations: a shape
function, the device kernel, and a ``cpu`` kernel in plain PyTorch for CPU
tensors (its lines 76-82 and 114-122), which the reference's own CPU tests call
through the op. The device selects the kernel: a GPU tensor never reaches the
``cpu`` one, and with ``libastrai_w8a8.so`` missing a GPU call raises. The
primitives this backend adds (``mm_fp8_bias``, ``linear_forward_fp8``, ...) are
device-only.
"""

from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
from torch import Tensor
from torch.library import custom_op

from astrai_amd.extension import loader

_FORMATS: Tuple[str, ...] = ("e4m3", "e5m2")
_OUTPUTS: Tuple[str, ...] = ("bf16", "e4m3")
_CODE_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)


class _Kernels:
    """The registry entry ``fp8_mm``, looked up on first use."""

    _entry = None

    @classmethod
    def get(cls):
        if cls._entry is None:
            entry = loader.get_module("fp8_mm") if loader.is_available("fp8_mm") else None
            if entry is None:
                raise RuntimeError(
                    "the 'fp8_mm' kernels are missing: libastrai_w8a8.so did not load "
                    "(build it with `make -C astrai_amd/csrc`)")
            cls._entry = entry
        return cls._entry


def _position(name: str, names: Sequence[str], what: str) -> int:
    if name not in names:
        raise ValueError(f"{what} must be one of {', '.join(map(repr, names))}; got {name!r}")
    return names.index(name)


def _all_bf16(what: str, *tensors: Tensor) -> None:
    bad = [str(t.dtype) for t in tensors if t.dtype != torch.bfloat16]
    if bad:
        raise TypeError(f"{what} takes bf16 tensors only (found {', '.join(bad)})")


def _device_only(op: str):
    raise RuntimeError(f"{op} has no CPU kernel in this backend: move the tensors to the GPU")


# ---------------------------------------------------------------------------
# dispatcher ops. Schemas are spelled out (they are the reference's, so traced
# graphs look the same); each op gets a shape function and a device kernel.
# ---------------------------------------------------------------------------

def _quantize_entry(x, scale, fmt):
    _device_only("custom::fp8_quantize")


def _quantize_host(x, scale, fmt):
    # CPU tensors only (reference ops/fp8.py:76-82): plain cast of x / step, floored amax
    codes = (x.float() / scale).to(_CODE_DTYPES[1 if fmt else 0])
    return codes, x.abs().amax().float().reshape(1).clamp_min(1e-12)


def _quantize_shapes(x, scale, fmt):
    codes = x.new_empty(x.shape, dtype=_CODE_DTYPES[1 if fmt else 0])
    return codes, x.new_empty(1, dtype=torch.float32)


def _quantize_device(x, scale, fmt):
    _all_bf16("custom::fp8_quantize", x)
    return _Kernels.get().quantize_bf16(x, scale, int(fmt))


def _gemm_entry(a, b, sa, sb, out_dtype=0, out_scale=None):
    _device_only("custom::fp8_gemm")


def _gemm_host(a, b, sa, sb, out_dtype=0, out_scale=None):
    # CPU tensors only (reference ops/fp8.py:114-122); the steps enter by broadcasting
    acc = a.float() @ b.float().t() * sa * sb
    if not out_dtype:
        return acc.to(torch.bfloat16)
    return (acc if out_scale is None else acc * out_scale).to(torch.float8_e4m3fn)


def _gemm_shapes(a, b, sa, sb, out_dtype=0, out_scale=None):
    return a.new_empty((a.shape[0], b.shape[0]),
                       dtype=torch.float8_e4m3fn if out_dtype else torch.bfloat16)


def _gemm_device(a, b, sa, sb, out_dtype=0, out_scale=None):
    if a.dtype not in _CODE_DTYPES or b.dtype != a.dtype:
        raise TypeError(f"custom::fp8_gemm takes two fp8 operands of one format (found {a.dtype} and {b.dtype})")
    return _Kernels.get().mm_fp8(a, b, sa, sb, int(out_dtype), out_scale)


fp8_quantize = custom_op("custom::fp8_quantize", _quantize_entry, mutates_args=(),
                         schema="(Tensor x, Tensor scale, int fmt) -> (Tensor, Tensor)")
fp8_quantize.register_fake(_quantize_shapes)
fp8_quantize.register_kernel("cuda")(_quantize_device)
fp8_quantize.register_kernel("cpu")(_quantize_host)

fp8_gemm = custom_op("custom::fp8_gemm", _gemm_entry, mutates_args=(),
                     schema="(Tensor a, Tensor b, Tensor sa, Tensor sb, int out_dtype=0, "
                            "Tensor? out_scale=None) -> Tensor")
fp8_gemm.register_fake(_gemm_shapes)
fp8_gemm.register_kernel("cuda")(_gemm_device)
fp8_gemm.register_kernel("cpu")(_gemm_host)


# ---------------------------------------------------------------------------
# the four primitives (string-level arguments) and this backend's additions
# ---------------------------------------------------------------------------

def quantize_bf16(x: Tensor, scale: Tensor, fmt: str = "e4m3"):
    """Codes of ``x / scale`` in the named fp8 format plus ``max |x|`` of the
    unscaled input, from one pass over ``x``. ``scale``: fp32 scalar on ``x``'s device."""
    return fp8_quantize(x, scale, _position(fmt, _FORMATS, "fmt"))


def mm_fp8(a: Tensor, b: Tensor, sa: Tensor, sb: Tensor, out_dtype: str = "bf16",
           out_scale: Optional[Tensor] = None) -> Tensor:
    """GEMM of fp8 codes ``a [M, K]`` and ``b [N, K]`` with fp32 accumulation, scaled by
    ``sa * sb``; as bf16, or as e4m3 codes of the result times ``out_scale``."""
    return fp8_gemm(a, b, sa, sb, _position(out_dtype, _OUTPUTS, "out_dtype"), out_scale)


def mm_fp8_bias(a: Tensor, b: Tensor, sa: Tensor, sb: Tensor, bias: Optional[Tensor]) -> Tensor:
    """``mm_fp8`` to bf16 with a bf16 ``bias [N]`` added in fp32 ahead of the one rounding:
    the epilogue order of the reference's fused forward (csrc/kernels/fp8/gemm.cuh:405-435)."""
    return _Kernels.get().mm_fp8(a, b, sa, sb, 0, None, bias)


def linear_forward_fp8(x: Tensor, w: Tensor, bias: Optional[Tensor], sx: Tensor, sw: Tensor):
    """``x @ w.T (+ bias)`` through e4m3 codes of both; also hands back the amax of ``x``
    and of ``w``. No bias: ``None``."""
    _all_bf16("linear_forward_fp8", x, w)
    no_bias = x.new_empty(0) if bias is None else bias  # the kernel entry wants a tensor
    return _Kernels.get().linear_forward_fp8(x, w, no_bias, sx, sw)


def linear_backward_fp8(g: Tensor, x: Tensor, w: Tensor, masks, sg: Tensor, sw: Tensor,
                        sx: Tensor, fmt: str = "e5m2"):
    """The three gradients of a linear layer from fp8 codes, which of them being chosen by
    ``masks`` (input, weight, bias), and the amax of ``g``."""
    _all_bf16("linear_backward_fp8", g, x, w)
    return _Kernels.get().linear_backward_fp8(g, x, w, [bool(m) for m in masks], sg, sw, sx,
                                              _position(fmt, _FORMATS, "fmt"))


def amax_bf16(x: Tensor) -> Tensor:
    """``max |x|`` of a bf16 device tensor as a fresh fp32 ``[1]`` tensor, one read of ``x``
    (what dynamic scaling measures before it can quantize)."""
    _all_bf16("amax_bf16", x)
    return _Kernels.get().amax_bf16(x)


def new_amax_partials(device) -> Tensor:
    """Scratch for the three ``*_partials`` primitives below: max |x| travels from the pass
    that sees the tensor to the ring push as one maximum per workgroup, not through one
    atomically updated (and beforehand cleared) slot. Producer and consumer share a stream."""
    return _Kernels.get().new_amax_partials(device)


def quantize_bf16_partials(x: Tensor, scale: Tensor, fmt: str, partials: Tensor) -> Tensor:
    """``quantize_bf16`` that leaves max |x| in ``partials`` and returns the codes alone."""
    _all_bf16("quantize_bf16_partials", x)
    return _Kernels.get().quantize_bf16_partials(x, scale, _position(fmt, _FORMATS, "fmt"), partials)


def amax_bf16_partials(x: Tensor, partials: Tensor) -> None:
    """``amax_bf16`` that leaves max |x| in ``partials``."""
    _all_bf16("amax_bf16_partials", x)
    _Kernels.get().amax_bf16_partials(x, partials)


def amax_ring_push_partials(hist: Tensor, idx: int, partials: Tensor, scale: Tensor, fmax: float,
                            pow2_margin: float, amax_out: Optional[Tensor] = None) -> None:
    """``amax_ring_push`` whose new amax is the maximum of ``partials`` (also written to
    ``amax_out`` when given)."""
    _Kernels.get().amax_ring_push_partials(hist, idx, partials, scale, fmax, pow2_margin, amax_out)


def amax_ring_push(hist: Tensor, idx: int, amax: Tensor, scale: Tensor, fmax: float,
                   pow2_margin: float) -> None:
    """Delayed scaling's bookkeeping for one tensor in one launch, in place: the new amax
    goes into slot ``idx`` of the ring, the scale becomes ``max(ring) / fmax / pow2_margin``."""
    _Kernels.get().amax_ring_push(hist, idx, amax, scale, fmax, pow2_margin)
