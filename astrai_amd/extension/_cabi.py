"""ctypes binding of ``lib/libastrai_w8a8.so`` (the C ABI in include/astrai_w8a8.h)
and the tensor-level adapters that stand where the reference's pybind module
``fp8_mm`` stands (csrc/kernels/fp8/mm.cu:350-369).

The adapters do what the reference binding does around its launches
(mm.cu:99-234): validate devices / dtypes / shapes, make operands contiguous,
allocate the outputs on the input's device, pass torch's current stream, and
turn a failing status into ``RuntimeError``. There is no CPU or PyTorch fallback
anywhere in this module: without the HIP library every call raises.
"""

from __future__ import annotations

import ctypes
import weakref
import os
from typing import Optional

import torch  # imported before the CDLL so the library binds to torch's HIP runtime

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
LIB_PATH = os.path.join(_LIB_DIR, "libastrai_w8a8.so")

ABI_VERSION = 1
OUT_BF16, OUT_E4M3, OUT_ACC = 0, 1, 2

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_INT = ctypes.c_int
_F32 = ctypes.c_float

# name -> argtypes, exactly the prototypes of include/astrai_w8a8.h
PROTOTYPES = {
    "astrai_w8a8_abi_version": ([], _INT),
    "astrai_w8a8_last_error": ([], ctypes.c_char_p),
    "astrai_w8a8_last_kernel": ([], ctypes.c_char_p),
    "astrai_w8a8_quantize_bf16_fp8": ([_P, _P, _P, _P, _I64, _INT, _P], _INT),
    "astrai_w8a8_amax_bf16": ([_P, _P, _I64, _P], _INT),
    "astrai_w8a8_amax_ring_push": ([_P, _INT, _INT, _P, _P, _F32, _F32, _P], _INT),
    "astrai_w8a8_quantize_bf16_fp8_partials": ([_P, _P, _P, _P, _I64, _INT, _P], _INT),
    "astrai_w8a8_amax_bf16_partials": ([_P, _P, _I64, _P], _INT),
    "astrai_w8a8_amax_ring_push_partials": ([_P, _INT, _INT, _P, _P, _P, _F32, _F32, _P], _INT),
    "astrai_w8a8_quantize_transpose_bf16_fp8": ([_P, _P, _P, _P, _P, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_quantize_bf16_int8_rows": ([_P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_add_rmsnorm_quantize_int8_rows": (
        [_P, _P, _P, ctypes.c_float, _P, _P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_silu_mul_quantize_int8_rows": ([_P, _P, _I64, _P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_add_rmsnorm_quantize_fp8_rows": (
        [_P, _P, _P, ctypes.c_float, _P, _P, _P, _P, _P, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_silu_mul_quantize_fp8_rows": ([_P, _P, _I64, _P, _P, _P, _P, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_mfma_probe": ([_INT, _P, _P, _P, _P], _INT),
    "astrai_w8a8_gemm_int8_ptpc_swiglu": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _INT),
    "astrai_w8a8_gemm_int8_ptpc_resid": ([_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _INT),
    "astrai_w8a8_quantize_int8_rows_pmax": ([_P, _P, _I64, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_silu_mul_quantize_int8_rows_blocked": ([_P, _I64, _I64, _P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_rope_cache_write_bf16": (
        [_P, _I64, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _P], _INT),
    "astrai_w8a8_attn_decode_workspace_floats": ([_I64, _I64, _I64, _I64], _I64),
    "astrai_w8a8_attn_paged_decode_bf16": (
        [_P, _P, _P, _P, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
         ctypes.c_float, _P], _INT),
    "astrai_w8a8_attn_paged_prefill_bf16": (
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _INT,
         ctypes.c_float, _P], _INT),
    "astrai_w8a8_rotary_emb_bf16": ([_P, _P, _P, _I64, _I64, _I64, _P], _INT),
    "astrai_w8a8_attn_paged_rows_workspace_floats": ([_I64, _I64, _I64, _I64, _I64, _INT], _I64),
    "astrai_w8a8_attn_paged_rows_bf16": (
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _P, _I64, _P, _I64, _I64,
         _I64, _I64, _I64, _I64, _I64, _INT, _I64, ctypes.c_float, _P], _INT),
    "astrai_w8a8_attn_paged_decode_masked_bf16": (
        [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _P, _I64, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
         _I64, ctypes.c_float, _P], _INT),
    "astrai_w8a8_attn_paged_prefill_masked_bf16": (
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _P, _I64, _I64, _I64, _I64,
         _I64, _I64, _I64, _INT, ctypes.c_float, _P], _INT),
    "astrai_w8a8_attn_prefill_bf16": (
        [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, ctypes.c_float, _P], _INT),
    "astrai_w8a8_attn_decode_bf16": (
        [_P, _P, _P, _P, _P, _I64, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, ctypes.c_float, _P],
        _INT),
    "astrai_w8a8_attn_decode_bf16_static_scratch": (
        [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, ctypes.c_float, _P], _INT),
    "astrai_w8a8_quantize_bf16_fp8_block128_act": ([_P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_quantize_bf16_fp8_block128_weight": ([_P, _P, _P, _I64, _I64, _P], _INT),
    "astrai_w8a8_gemm_fp8_pt": ([_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _INT, _INT, _P], _INT),
    "astrai_w8a8_gemm_fp8_ptpc": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_gemm_fp8_block128": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P], _INT),
    "astrai_w8a8_gemm_int8_ptpc": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_gemv_int8_ptpc": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_gemm_int8_ptpc_tiled": ([_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _INT, _P], _INT),
    "astrai_w8a8_gemm_int8_ptpc_rope_cache": (
        [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _P], _INT),
}

_lib: Optional[ctypes.CDLL] = None
_load_error: Optional[str] = None


def load() -> Optional[ctypes.CDLL]:
    """Load the shared library once; ``None`` (with the reason kept) if it is absent
    or does not carry the expected ABI. Never raises: the registry reports an
    unavailable kernel the way the reference's loader does (loader.py:36-44)."""
    global _lib, _load_error
    if _lib is not None or _load_error is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        _load_error = f"{LIB_PATH} not built"
        return None
    try:
        lib = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        got = lib.astrai_w8a8_abi_version()
        if got != ABI_VERSION:
            raise OSError(f"ABI version {got}, expected {ABI_VERSION}")
    except (OSError, AttributeError) as e:
        _load_error = f"{type(e).__name__}: {e}"
        return None
    _lib = lib
    return _lib


def load_error() -> Optional[str]:
    return _load_error


def _require() -> ctypes.CDLL:
    lib = load()
    if lib is None:
        raise RuntimeError(
            f"HIP library libastrai_w8a8.so is not available ({_load_error}). "
            "Build it with `make -C astrai_amd/csrc`."
        )
    return lib


def _check(rc: int, lib: ctypes.CDLL) -> None:
    if rc != 0:
        msg = lib.astrai_w8a8_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"astrai_w8a8 error {rc}: {msg}")


try:  # the raw handle of the current stream without building a Stream object (a microsecond per call saved)
    from torch._C import _cuda_getCurrentRawStream as _raw_stream
except ImportError:  # pragma: no cover
    _raw_stream = None


def _stream(t: torch.Tensor) -> int:
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device(dev: torch.device):
    """``torch.cuda.device(dev)``, or nothing when ``dev`` is the current device already (every
    call of a single-GPU process): the guard object costs more than a launch on the decode path."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(dev)


# Rows that are not whole 16-byte pieces (K % 16 != 0) cannot be fetched by the tiled kernels'
# 16-byte loads, and the any-shape kernel they would take instead runs at ~14 TOP/s (a 4096 x
# 4096 x 4104 product: 9.7 ms against 0.1 ms). Zero columns change no sum, so from this many
# multiply-adds on both operands are copied into rows padded with zero codes.
_PAD_K_MIN_MACS = 1 << 24


# padded forms of weight-side operands: key -> (weakref to the operand, its version, padded copy).
# A Linear's codes are one long-lived tensor (Int8State, the fp8 weight metas), so its padded form
# is made once, not on every call; an entry dies with its tensor or with a write to it.
_padded_weights: dict = {}


def _padded_weight(b_c: torch.Tensor, kp: int) -> torch.Tensor:
    key = (b_c.data_ptr(), tuple(b_c.shape), b_c.dtype, kp)
    hit = _padded_weights.get(key)
    if hit is not None and hit[0]() is b_c and hit[1] == b_c._version:
        return hit[2]
    for dead in [k_ for k_, e in _padded_weights.items() if e[0]() is None]:
        del _padded_weights[dead]
    padded = torch.nn.functional.pad(b_c.view(torch.uint8), (0, kp - b_c.size(1))).view(b_c.dtype)
    _padded_weights[key] = (weakref.ref(b_c), b_c._version, padded)
    return padded


def _pad_k(a_c: torch.Tensor, b_c: torch.Tensor):
    """``(a, b, k)`` with K padded by zero codes to the next multiple the tuned kernels take (256 for
    at most 128 activation rows, the decode kernels' item; 128 otherwise), when K % 16 != 0 and the
    product is large enough to repay the copies; else the operands as they are. The activation is
    padded per call; the weight-side operand's padded form is kept while that tensor lives unmodified."""
    m, k = a_c.shape
    n = b_c.size(0)
    if k % 16 == 0 or m * n * k < _PAD_K_MIN_MACS:
        return a_c, b_c, k
    q = 256 if m <= 128 else 128
    kp = -(-k // q) * q
    a_p = torch.nn.functional.pad(a_c.view(torch.uint8), (0, kp - k)).view(a_c.dtype)
    return a_p, _padded_weight(b_c, kp), kp


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name}: CUDA tensors required")  # mm.cu:104,135,192


def _check_scale(scale: torch.Tensor, ref: torch.Tensor, name: str) -> None:
    # mm.cu:49-54
    if not (scale.is_cuda and scale.device == ref.device and scale.dtype == torch.float32
            and scale.numel() == 1):
        raise RuntimeError(f"{name} must be a CUDA float32 scalar on the input device")


def _check_vec(s: torch.Tensor, ref: torch.Tensor, numel: int, name: str) -> torch.Tensor:
    if not (s.is_cuda and s.device == ref.device and s.dtype == torch.float32
            and s.numel() == numel):
        raise RuntimeError(f"{name} must be CUDA float32 with {numel} elements on the input device")
    return s.contiguous()


_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)


# ---------------------------------------------------------------------------
# The five callables of the reference's pybind module (mm.cu:350-369)
# ---------------------------------------------------------------------------


def quantize_bf16(x: torch.Tensor, scale: torch.Tensor, fmt: int):
    """bf16 -> fp8 with fused amax; returns ``(x8, amax)``. mm.cu:99-126."""
    lib = _require()
    _gpu(x, "quantize_bf16")
    _gpu(scale, "quantize_bf16")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    _check_scale(scale, x, "scale")
    x_c = x.contiguous()
    with _on_device(x.device):
        x8 = torch.empty_like(x_c, dtype=torch.float8_e5m2 if fmt else torch.float8_e4m3fn)
        amax = torch.zeros(1, device=x.device, dtype=torch.float32)
        if x_c.numel():
            _check(lib.astrai_w8a8_quantize_bf16_fp8(
                x_c.data_ptr(), x8.data_ptr(), scale.data_ptr(), amax.data_ptr(),
                x_c.numel(), 1 if fmt else 0, _stream(x)), lib)
    return x8, amax


def mm_fp8(a: torch.Tensor, b: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor,
           out_dtype: int = 0, out_scale: Optional[torch.Tensor] = None,
           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Pre-quantized fp8 GEMM ``a @ b^T * sa * sb``. mm.cu:128-184. ``bias`` (bf16
    ``[N]``, bf16 output only) is an extension used by the fused linear forward.
    Scales are fp32 scalars, as the reference's binding demands (mm.cu:49-54) -- or,
    for bf16 output, the shapes its CPU kernel's broadcast accepts besides
    (ops/fp8.py:118): ``sa`` one step per activation row (``[M]`` / ``[M, 1]``) and / or
    ``sb`` one per weight row (``[N]`` / ``[1, N]``)."""
    lib = _require()
    _gpu(a, "mm_fp8")
    _gpu(b, "mm_fp8")
    if a.dtype not in _FP8:
        raise RuntimeError("a and b must be fp8 (e4m3fn or e5m2)")
    if a.dtype != b.dtype:
        raise RuntimeError("a and b must share the same fp8 format")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("a and b must be 2D")
    if a.device != b.device:
        raise RuntimeError("a and b must be on the same device")
    if a.size(1) != b.size(1):
        raise RuntimeError("inner dim mismatch")
    per_row = ((sa.numel() > 1 and tuple(sa.shape) in ((a.size(0),), (a.size(0), 1)))
               or (sb.numel() > 1 and tuple(sb.shape) in ((b.size(0),), (1, b.size(0)))))
    per_row = per_row and out_dtype == 0
    if not per_row or sa.numel() == 1:
        _check_scale(sa, a, "sa")
    if not per_row or sb.numel() == 1:
        _check_scale(sb, a, "sb")
    if out_dtype not in (0, 1):
        raise RuntimeError("out_dtype must be 0 (bf16) or 1 (fp8 e4m3)")
    if out_dtype == 1:
        if out_scale is None:
            raise RuntimeError("fp8 output requires out_scale")
        _check_scale(out_scale, a, "out_scale")
    a_c, b_c = a.contiguous(), b.contiguous()
    m, k = a_c.shape
    n = b_c.size(0)
    if bias is not None:
        if not (bias.is_cuda and bias.device == a.device and bias.dtype == torch.bfloat16
                and bias.numel() == n):
            raise RuntimeError("bias must be CUDA bf16 with shape [N]")
        bias = bias.contiguous()
    with _on_device(a.device):
        a_c, b_c, k = _pad_k(a_c, b_c)
        out = torch.empty((m, n), device=a.device,
                          dtype=torch.float8_e4m3fn if out_dtype else torch.bfloat16)
        if m and n:
            if k == 0:  # an empty sum: zeros (plus the bias)
                out.zero_()
                if bias is not None:
                    out.copy_(bias.expand(m, n))
            elif per_row:
                sa_v = _check_vec(sa.reshape(-1).expand(m) if sa.numel() == 1 else sa.reshape(-1), a, m, "sa")
                sb_v = _check_vec(sb.reshape(-1).expand(n) if sb.numel() == 1 else sb.reshape(-1), a, n, "sb")
                _check(lib.astrai_w8a8_gemm_fp8_ptpc(
                    a_c.data_ptr(), b_c.data_ptr(), sa_v.data_ptr(), sb_v.data_ptr(), _ptr(bias),
                    out.data_ptr(), m, n, k, 1 if a.dtype == torch.float8_e5m2 else 0, _stream(a)), lib)
            else:
                _check(lib.astrai_w8a8_gemm_fp8_pt(
                    a_c.data_ptr(), b_c.data_ptr(), sa.data_ptr(), sb.data_ptr(),
                    _ptr(out_scale) if out_dtype else None, _ptr(bias), out.data_ptr(),
                    m, n, k, 1 if a.dtype == torch.float8_e5m2 else 0, out_dtype, _stream(a)), lib)
    return out


def mm_fp8_acc(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Raw fp32 accumulator of the fp8 GEMM (parity surface, no scaling)."""
    lib = _require()
    a_c, b_c = a.contiguous(), b.contiguous()
    m, k = a_c.shape
    n = b_c.size(0)
    with _on_device(a.device):
        out = torch.empty((m, n), device=a.device, dtype=torch.float32)
        _check(lib.astrai_w8a8_gemm_fp8_pt(
            a_c.data_ptr(), b_c.data_ptr(), None, None, None, None, out.data_ptr(), m, n, k,
            1 if a.dtype == torch.float8_e5m2 else 0, OUT_ACC, _stream(a)), lib)
    return out


def linear_forward_fp8(x: torch.Tensor, w: torch.Tensor, bias: torch.Tensor,
                       sx: torch.Tensor, sw: torch.Tensor):
    """bf16 linear forward through e4m3: returns ``(out, amax_x, amax_w)``.
    mm.cu:186-234. The reference re-quantizes both operands inside its GEMM at
    every K step (gemm.cuh:296-326); here each operand is quantized once by the
    prologue kernel (which also yields its amax) and the pre-quantized MFMA GEMM
    applies ``sx*sw`` and the bias in its epilogue -- the same arithmetic."""
    _gpu(x, "linear_forward_fp8")
    _gpu(w, "linear_forward_fp8")
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise RuntimeError("x and w must be bf16")
    if x.device != w.device:
        raise RuntimeError("x and w must be on the same device")
    _check_scale(sx, x, "sx")
    _check_scale(sw, x, "sw")
    if w.dim() != 2 or x.size(-1) != w.size(1):
        raise RuntimeError("inner dim mismatch")
    k, n = w.size(1), w.size(0)
    x2 = x.reshape(-1, k)
    has_bias = bias is not None and bias.numel() > 0
    if has_bias and not (bias.is_cuda and bias.device == x.device
                         and bias.dtype == torch.bfloat16 and bias.numel() == n):
        raise RuntimeError("bias must be CUDA bf16 with shape [N]")
    x8, amax_x = quantize_bf16(x2, sx, 0)
    w8, amax_w = quantize_bf16(w, sw, 0)
    out = mm_fp8(x8, w8, sx, sw, 0, None, bias if has_bias else None)
    return out.reshape(*x.shape[:-1], n), amax_x, amax_w


def fp8_mm(a: torch.Tensor, b: torch.Tensor, sx: torch.Tensor, sw: torch.Tensor) -> torch.Tensor:
    """bf16-in fused fp8 GEMM primitive (no bias, no amax). mm.cu:322-348."""
    _gpu(a, "fp8_mm")
    _gpu(b, "fp8_mm")
    if a.dtype != torch.bfloat16 or b.dtype != torch.bfloat16:
        raise RuntimeError("a and b must be bf16")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("a and b must be 2D")
    if a.device != b.device:
        raise RuntimeError("a and b must be on the same device")
    if a.size(1) != b.size(1):
        raise RuntimeError("inner dim mismatch")
    out, _, _ = linear_forward_fp8(a, b, None, sx, sw)
    return out


def amax_bf16(x: torch.Tensor) -> torch.Tensor:
    """``x.abs().amax()`` of a bf16 tensor as fp32 ``[1]`` from one read of ``x``
    (the measurement of dynamic scaling, astrai/extension/fp8.py:289-292)."""
    lib = _require()
    _gpu(x, "amax_bf16")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    x_c = x.contiguous()
    with _on_device(x.device):
        amax = torch.zeros(1, device=x.device, dtype=torch.float32)
        if x_c.numel():
            _check(lib.astrai_w8a8_amax_bf16(x_c.data_ptr(), amax.data_ptr(), x_c.numel(),
                                            _stream(x)), lib)
    return amax


def amax_ring_push(hist: torch.Tensor, idx: int, amax: torch.Tensor, scale: torch.Tensor,
                   fmax: float, pow2_margin: float) -> None:
    """In place: ``hist[idx] = amax; scale = max((hist.max() / fmax) / pow2_margin, 1e-12)``
    (FP8TensorMeta's record-then-refresh, astrai/extension/fp8.py:147-173)."""
    lib = _require()
    _gpu(hist, "amax_ring_push")
    for t, name in ((hist, "hist"), (amax, "amax"), (scale, "scale")):
        if not (t.is_cuda and t.device == hist.device and t.dtype == torch.float32
                and t.is_contiguous()):
            raise RuntimeError(f"{name} must be a contiguous float32 tensor on the ring's device")
    if amax.numel() != 1 or scale.numel() != 1:
        raise RuntimeError("amax and scale must have one element")
    with _on_device(hist.device):
        _check(lib.astrai_w8a8_amax_ring_push(hist.data_ptr(), hist.numel(), int(idx),
                                             amax.data_ptr(), scale.data_ptr(), float(fmax),
                                             float(pow2_margin), _stream(hist)), lib)


AMAX_PARTIALS = 1024   # ASTRAI_W8A8_AMAX_PARTIALS


def new_amax_partials(device) -> torch.Tensor:
    """A zeroed array for the per-workgroup maxima of :func:`quantize_bf16_partials` /
    :func:`amax_bf16_partials` (producer and consumer must run on one stream)."""
    return torch.zeros(AMAX_PARTIALS, device=device, dtype=torch.float32)


def _check_partials(partials: torch.Tensor, ref: torch.Tensor) -> None:
    if not (partials.is_cuda and partials.device == ref.device and partials.dtype == torch.float32
            and partials.numel() == AMAX_PARTIALS and partials.is_contiguous()):
        raise RuntimeError(f"partials must be a contiguous float32 tensor of {AMAX_PARTIALS} elements on the input device")


def quantize_bf16_partials(x: torch.Tensor, scale: torch.Tensor, fmt: int, partials: torch.Tensor) -> torch.Tensor:
    """:func:`quantize_bf16` with max |x| left as per-workgroup maxima in ``partials`` (every
    slot written) for :func:`amax_ring_push_partials`; returns the codes."""
    lib = _require()
    _gpu(x, "quantize_bf16_partials")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    _check_scale(scale, x, "scale")
    _check_partials(partials, x)
    x_c = x.contiguous()
    with _on_device(x.device):
        x8 = torch.empty_like(x_c, dtype=torch.float8_e5m2 if fmt else torch.float8_e4m3fn)
        if x_c.numel():
            _check(lib.astrai_w8a8_quantize_bf16_fp8_partials(
                x_c.data_ptr(), x8.data_ptr(), scale.data_ptr(), partials.data_ptr(),
                x_c.numel(), 1 if fmt else 0, _stream(x)), lib)
        else:
            partials.zero_()
    return x8


def amax_bf16_partials(x: torch.Tensor, partials: torch.Tensor) -> None:
    """max |x| of a bf16 tensor as per-workgroup maxima in ``partials`` (every slot written)."""
    lib = _require()
    _gpu(x, "amax_bf16_partials")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    _check_partials(partials, x)
    x_c = x.contiguous()
    with _on_device(x.device):
        if x_c.numel():
            _check(lib.astrai_w8a8_amax_bf16_partials(x_c.data_ptr(), partials.data_ptr(), x_c.numel(),
                                                     _stream(x)), lib)
        else:
            partials.zero_()


def amax_ring_push_partials(hist: torch.Tensor, idx: int, partials: torch.Tensor, scale: torch.Tensor,
                            fmax: float, pow2_margin: float, amax_out: Optional[torch.Tensor] = None) -> None:
    """:func:`amax_ring_push` with the fresh amax taken as the maximum of ``partials``."""
    lib = _require()
    _gpu(hist, "amax_ring_push_partials")
    for t, name in ((hist, "hist"), (scale, "scale")) + (((amax_out, "amax_out"),) if amax_out is not None else ()):
        if not (t.is_cuda and t.device == hist.device and t.dtype == torch.float32 and t.is_contiguous()):
            raise RuntimeError(f"{name} must be a contiguous float32 tensor on the ring's device")
    _check_partials(partials, hist)
    if scale.numel() != 1 or (amax_out is not None and amax_out.numel() != 1):
        raise RuntimeError("scale and amax_out must have one element")
    with _on_device(hist.device):
        _check(lib.astrai_w8a8_amax_ring_push_partials(
            hist.data_ptr(), hist.numel(), int(idx), partials.data_ptr(), _ptr(amax_out), scale.data_ptr(),
            float(fmax), float(pow2_margin), _stream(hist)), lib)


def quantize_transpose_bf16(x: torch.Tensor, scale: torch.Tensor, fmt: int,
                            want_rowmajor: bool = False, want_amax: bool = False):
    """One pass over a bf16 ``[R, C]`` matrix -> ``(x8 [R,C] or None, x8t [C,R], amax [1] or None)``:
    the codes ``quantize_bf16`` gives for ``x`` and for ``x.t().contiguous()``
    (mm.cu:276-312 makes that copy first). ``amax`` is measured (and its slot allocated and
    cleared: one more launch) only when asked for."""
    lib = _require()
    _gpu(x, "quantize_transpose_bf16")
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise RuntimeError("x must be a 2D bf16 tensor")
    _check_scale(scale, x, "scale")
    x_c = x.contiguous()
    rows, cols = x_c.shape
    f8 = torch.float8_e5m2 if fmt else torch.float8_e4m3fn
    with _on_device(x.device):
        x8 = torch.empty((rows, cols), device=x.device, dtype=f8) if want_rowmajor else None
        x8t = torch.empty((cols, rows), device=x.device, dtype=f8)
        amax = torch.zeros(1, device=x.device, dtype=torch.float32) if want_amax else None
        if rows and cols:
            _check(lib.astrai_w8a8_quantize_transpose_bf16_fp8(
                x_c.data_ptr(), _ptr(x8), x8t.data_ptr(), scale.data_ptr(),
                _ptr(amax), rows, cols, 1 if fmt else 0, _stream(x)), lib)
    return x8, x8t, amax


def _mm_fp8_into(out: torch.Tensor, a8: torch.Tensor, b8: torch.Tensor, sa, sb, lib):
    m, k = a8.shape
    n = b8.size(0)
    if not (m and n):
        return
    if k == 0:
        out.zero_()
        return
    _check(lib.astrai_w8a8_gemm_fp8_pt(
        a8.data_ptr(), b8.data_ptr(), sa.data_ptr(), sb.data_ptr(), None, None, out.data_ptr(),
        m, n, k, 1 if a8.dtype == torch.float8_e5m2 else 0, 0, _stream(a8)), lib)


def linear_backward_fp8(g, x, w, masks, sg, sw, sx, fmt: int):
    """FP8 linear backward ``(grad_input, grad_weight, grad_bias, amax_g)``.
    mm.cu:236-320: ``dX = g8 @ w8`` and ``dW = g8^T @ x8`` as NT GEMMs. The
    reference copies g, w and x transposed and quantizes each copy; here one
    kernel per tensor reads it once and writes the codes in the layouts the two
    GEMMs contract over (g in both), and the GEMMs write the gradients in place."""
    lib = _require()
    _gpu(g, "linear_backward_fp8")
    if not (g.dtype == x.dtype == w.dtype == torch.bfloat16):
        raise RuntimeError("g, x, and w must be bf16")
    if not (g.device == x.device == w.device):
        raise RuntimeError("g, x, and w must be on the same device")
    masks = list(masks)
    if len(masks) != 3:
        raise RuntimeError("masks must contain three values")
    n, k = w.shape
    g_c = g.reshape(-1, n).contiguous()
    x_c = x.reshape(-1, x.size(-1)).contiguous()
    m = g_c.size(0)
    if x_c.size(0) != m or x_c.size(1) != k:
        raise RuntimeError("backward shape mismatch")
    for t, name in ((sg, "sg"), (sw, "sw"), (sx, "sx")):
        _check_scale(t, g, name)
    with _on_device(g.device):
        grad_input = torch.empty(x.shape, device=x.device, dtype=x.dtype)
        grad_weight = torch.empty((n, k), device=w.device, dtype=w.dtype)
        grad_bias = torch.empty(0, device=g.device, dtype=g.dtype)
        amax_g = None
        g8 = g8_t = None
        if masks[1]:
            # amax_g is measured only on the dX branch (mm.cu:293-296)
            g8, g8_t, amax = quantize_transpose_bf16(g_c, sg, fmt, want_rowmajor=bool(masks[0]),
                                                     want_amax=bool(masks[0]))
            if masks[0]:
                amax_g = amax
        elif masks[0]:
            g8, amax_g = quantize_bf16(g_c, sg, fmt)
        if masks[0]:
            _, w8_t, _ = quantize_transpose_bf16(w, sw, fmt)  # [K, N]
            _mm_fp8_into(grad_input, g8, w8_t, sg, sw, lib)
        if masks[1]:
            _, x8_t, _ = quantize_transpose_bf16(x_c, sx, fmt)  # [K, M]
            _mm_fp8_into(grad_weight, g8_t, x8_t, sg, sx, lib)
        if not masks[0] and not masks[1]:
            amax_g = g_c.abs().amax().to(torch.float32).reshape(1)
        if masks[2]:
            grad_bias = g_c.sum(0).to(g.dtype)
        if amax_g is None:
            amax_g = torch.zeros(1, device=g.device, dtype=torch.float32)
    return grad_input, grad_weight, grad_bias, amax_g


# ---------------------------------------------------------------------------
# int8 per-token x per-channel and 128-block fp8 (not in the reference)
# ---------------------------------------------------------------------------


def quantize_int8_rows(x: torch.Tensor):
    """bf16 ``[..., K]`` -> ``(xq int8 [R,K], s fp32 [R,1])``, one symmetric scale per row."""
    lib = _require()
    _gpu(x, "quantize_int8_rows")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    if x.dim() < 1:
        raise RuntimeError("x must have at least one dimension")
    k = x.size(-1)
    x2 = x.reshape(-1, k).contiguous()
    rows = x2.size(0)
    with _on_device(x.device):
        xq = torch.empty((rows, k), device=x.device, dtype=torch.int8)
        s = torch.empty((rows, 1), device=x.device, dtype=torch.float32)
        if rows and k:
            _check(lib.astrai_w8a8_quantize_bf16_int8_rows(
                x2.data_ptr(), xq.data_ptr(), s.data_ptr(), rows, k, _stream(x)), lib)
        elif rows:
            s.fill_(1e-12 / 127.0)
    return xq, s


def add_rmsnorm_quantize_int8(x: torch.Tensor, weight: torch.Tensor, eps: float,
                              res: Optional[torch.Tensor] = None, want_y: bool = False):
    """``t = x + res`` (bf16, when ``res`` is given), ``y = rms_norm(t) * weight``, per-row
    int8 of ``y`` in one kernel. Returns ``(xq [R,K], s [R,1], t or None, y or None)``."""
    lib = _require()
    _gpu(x, "add_rmsnorm_quantize_int8")
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("x and weight must be bf16")
    k = x.size(-1)
    if weight.numel() != k or weight.device != x.device:
        raise RuntimeError("weight must be [K] on x's device")
    x2 = x.reshape(-1, k).contiguous()
    rows = x2.size(0)
    r2 = None
    if res is not None:
        if res.shape != x.shape or res.dtype != torch.bfloat16 or res.device != x.device:
            raise RuntimeError("res must match x in shape, dtype and device")
        r2 = res.reshape(-1, k).contiguous()
    with _on_device(x.device):
        xq = torch.empty((rows, k), device=x.device, dtype=torch.int8)
        s = torch.empty((rows, 1), device=x.device, dtype=torch.float32)
        t = torch.empty_like(x2) if r2 is not None else None
        y = torch.empty_like(x2) if want_y else None
        _check(lib.astrai_w8a8_add_rmsnorm_quantize_int8_rows(
            x2.data_ptr(), _ptr(r2), weight.contiguous().data_ptr(), float(eps), _ptr(t), _ptr(y),
            xq.data_ptr(), s.data_ptr(), rows, k, _stream(x)), lib)
    return (xq, s, None if t is None else t.reshape(x.shape), None if y is None else y.reshape(x.shape))


def silu_mul_quantize_int8(gate: torch.Tensor, up: torch.Tensor, want_h: bool = False):
    """``h = up * silu(gate)`` (bf16 arithmetic) and per-row int8 of ``h`` in one kernel.
    ``gate`` / ``up`` are ``[..., W]`` views whose last dimension is contiguous and whose
    rows are equally spaced (e.g. the two halves of a ``[R, 2W]`` tensor).
    Returns ``(hq [R,W], s [R,1], h or None)``."""
    lib = _require()
    _gpu(gate, "silu_mul_quantize_int8")
    if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16:
        raise RuntimeError("gate and up must be bf16")
    if gate.shape != up.shape or gate.device != up.device:
        raise RuntimeError("gate and up must match in shape and device")
    w = gate.size(-1)
    g2, u2 = gate.reshape(-1, w), up.reshape(-1, w)
    if g2.stride(1) != 1 or u2.stride(1) != 1 or g2.stride(0) != u2.stride(0):
        g2, u2 = g2.contiguous(), u2.contiguous()
    rows = g2.size(0)
    ld = g2.stride(0) if rows > 1 else max(w, g2.stride(0))
    with _on_device(gate.device):
        hq = torch.empty((rows, w), device=gate.device, dtype=torch.int8)
        s = torch.empty((rows, 1), device=gate.device, dtype=torch.float32)
        h = torch.empty((rows, w), device=gate.device, dtype=torch.bfloat16) if want_h else None
        _check(lib.astrai_w8a8_silu_mul_quantize_int8_rows(
            g2.data_ptr(), u2.data_ptr(), ld, _ptr(h), hq.data_ptr(), s.data_ptr(), rows, w,
            _stream(gate)), lib)
    return hq, s, None if h is None else h.reshape(gate.shape)


def _fp8_scale_amax(scale: torch.Tensor, amax: Optional[torch.Tensor], ref: torch.Tensor):
    if not (scale.is_cuda and scale.device == ref.device and scale.dtype == torch.float32
            and scale.numel() == 1):
        raise RuntimeError("scale must be one CUDA float32 on the input device")
    if amax is not None and not (amax.is_cuda and amax.device == ref.device
                                 and amax.dtype == torch.float32 and amax.numel() == 1):
        raise RuntimeError("amax must be one CUDA float32 on the input device")


def add_rmsnorm_quantize_fp8(x: torch.Tensor, weight: torch.Tensor, eps: float, scale: torch.Tensor,
                             res: Optional[torch.Tensor] = None, fmt: int = 0,
                             amax: Optional[torch.Tensor] = None, want_y: bool = False):
    """Per-tensor fp8 twin of :func:`add_rmsnorm_quantize_int8` for a step known ahead
    (delayed scaling): ``(x8 [R,K] fp8, amax [1], t or None, y or None)``; ``amax`` (a zeroed
    slot is made when none is given) ends as ``max(amax, max |y|)``."""
    lib = _require()
    _gpu(x, "add_rmsnorm_quantize_fp8")
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("x and weight must be bf16")
    k = x.size(-1)
    if weight.numel() != k or weight.device != x.device:
        raise RuntimeError("weight must be [K] on x's device")
    _fp8_scale_amax(scale, amax, x)
    x2 = x.reshape(-1, k).contiguous()
    rows = x2.size(0)
    r2 = None
    if res is not None:
        if res.shape != x.shape or res.dtype != torch.bfloat16 or res.device != x.device:
            raise RuntimeError("res must match x in shape, dtype and device")
        r2 = res.reshape(-1, k).contiguous()
    with _on_device(x.device):
        x8 = torch.empty((rows, k), device=x.device, dtype=_FP8[1 if fmt else 0])
        if amax is None:
            amax = torch.zeros(1, device=x.device, dtype=torch.float32)
        t = torch.empty_like(x2) if r2 is not None else None
        y = torch.empty_like(x2) if want_y else None
        _check(lib.astrai_w8a8_add_rmsnorm_quantize_fp8_rows(
            x2.data_ptr(), _ptr(r2), weight.contiguous().data_ptr(), float(eps), _ptr(t), _ptr(y),
            x8.data_ptr(), scale.data_ptr(), amax.data_ptr(), rows, k, 1 if fmt else 0, _stream(x)), lib)
    return (x8, amax, None if t is None else t.reshape(x.shape), None if y is None else y.reshape(x.shape))


def silu_mul_quantize_fp8(gate: torch.Tensor, up: torch.Tensor, scale: torch.Tensor, fmt: int = 0,
                          amax: Optional[torch.Tensor] = None, want_h: bool = False):
    """Per-tensor fp8 twin of :func:`silu_mul_quantize_int8`: ``(h8 [R,W] fp8, amax [1], h or
    None)``."""
    lib = _require()
    _gpu(gate, "silu_mul_quantize_fp8")
    if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16:
        raise RuntimeError("gate and up must be bf16")
    if gate.shape != up.shape or gate.device != up.device:
        raise RuntimeError("gate and up must match in shape and device")
    _fp8_scale_amax(scale, amax, gate)
    w = gate.size(-1)
    g2, u2 = gate.reshape(-1, w), up.reshape(-1, w)
    if g2.stride(1) != 1 or u2.stride(1) != 1 or g2.stride(0) != u2.stride(0):
        g2, u2 = g2.contiguous(), u2.contiguous()
    rows = g2.size(0)
    ld = g2.stride(0) if rows > 1 else max(w, g2.stride(0))
    with _on_device(gate.device):
        h8 = torch.empty((rows, w), device=gate.device, dtype=_FP8[1 if fmt else 0])
        if amax is None:
            amax = torch.zeros(1, device=gate.device, dtype=torch.float32)
        h = torch.empty((rows, w), device=gate.device, dtype=torch.bfloat16) if want_h else None
        _check(lib.astrai_w8a8_silu_mul_quantize_fp8_rows(
            g2.data_ptr(), u2.data_ptr(), ld, _ptr(h), h8.data_ptr(), scale.data_ptr(), amax.data_ptr(),
            rows, w, 1 if fmt else 0, _stream(gate)), lib)
    return h8, amax, None if h is None else h.reshape(gate.shape)


def rotary_emb(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    """Rotate adjacent pairs of ``x`` (bf16, packed ``[tokens, heads, head_dim]`` or dense
    ``[batch, seq, heads, head_dim]``) by ``freqs_cis`` (fp32, the same token axes followed by
    ``[head_dim/2, 2]`` = cos, sin); a new tensor of ``x``'s shape. Argument checks and
    messages of the reference's entry (csrc/kernels/rotary/rotary_emb.cu:47-93)."""
    lib = _require()
    if not x.is_cuda:
        raise RuntimeError("x must be on CUDA")
    if not freqs_cis.is_cuda:
        raise RuntimeError("freqs_cis must be on CUDA")
    if x.dtype != torch.bfloat16:
        raise RuntimeError("x must be bf16")
    if x.dim() not in (3, 4):
        raise RuntimeError("x must be [tokens, n_heads, head_dim] or [batch, seq_len, n_heads, head_dim]")
    if not x.is_contiguous():
        raise RuntimeError("x must be contiguous")
    if freqs_cis.dim() != x.dim():
        raise RuntimeError("freqs_cis rank must match x rank")
    if not freqs_cis.is_contiguous():
        raise RuntimeError("freqs_cis must be contiguous")
    if freqs_cis.dtype != torch.float32:
        raise RuntimeError("freqs_cis must be f32")
    if freqs_cis.device != x.device:
        raise RuntimeError("freqs_cis must be on x's device")
    tokens = x.size(0) if x.dim() == 3 else x.size(0) * x.size(1)
    heads, head_dim = x.size(-2), x.size(-1)
    if head_dim % 2:
        raise RuntimeError("head_dim must be even")
    if freqs_cis.numel() != tokens * head_dim:
        raise RuntimeError("freqs_cis token or rotary dimension mismatch")
    if freqs_cis.size(-2) != head_dim // 2:
        raise RuntimeError("freqs_cis dim/2 mismatch")
    if freqs_cis.size(-1) != 2:
        raise RuntimeError("freqs_cis last dim must be 2 [cos, sin]")
    with _on_device(x.device):
        out = torch.empty_like(x)
        if x.numel():
            _check(lib.astrai_w8a8_rotary_emb_bf16(x.data_ptr(), freqs_cis.data_ptr(), out.data_ptr(),
                                                   tokens, heads, head_dim, _stream(x)), lib)
    return out


def rope_cache_write(qkv: torch.Tensor, freqs: torch.Tensor, positions: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, n_heads: int, n_kv_heads: int,
                     head_dim: int) -> torch.Tensor:
    """Rotate q and k of ``qkv [batch, seq, (n_heads + 2 n_kv_heads) * head_dim]`` (a view whose
    last dimension is contiguous and whose tokens are equally spaced), write k and v into
    ``k_cache`` / ``v_cache`` ``[batch, n_kv_heads, max_len, head_dim]`` at ``positions [seq]``
    and return q as ``[batch, n_heads, seq, head_dim]``. ``freqs`` is fp32
    ``[seq, head_dim/2, 2]`` (cos, sin)."""
    lib = _require()
    _gpu(qkv, "rope_cache_write")
    if qkv.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("qkv and the caches must be bf16")
    if qkv.dim() != 3:
        raise RuntimeError("qkv must be [batch, seq, features]")
    b, s, feat = qkv.shape
    if feat != (n_heads + 2 * n_kv_heads) * head_dim:
        raise RuntimeError("qkv features must be (n_heads + 2 n_kv_heads) * head_dim")
    q2 = qkv.reshape(b * s, feat)
    if q2.stride(1) != 1:
        q2 = q2.contiguous()
    ld = q2.stride(0) if b * s > 1 else max(feat, q2.stride(0))
    if freqs.dtype != torch.float32 or tuple(freqs.shape[-3:]) != (s, head_dim // 2, 2):
        raise RuntimeError("freqs must be fp32 [seq, head_dim/2, 2]")
    if positions.dtype != torch.int64 or positions.numel() != s:
        raise RuntimeError("positions must be int64 [seq]")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()) or k_cache.shape != v_cache.shape:
        raise RuntimeError("caches must be contiguous and of one shape")
    if k_cache.dim() != 4 or k_cache.size(0) != b or k_cache.size(1) != n_kv_heads or k_cache.size(3) != head_dim:
        raise RuntimeError("caches must be [batch, n_kv_heads, max_len, head_dim]")
    for t in (freqs, positions, k_cache, v_cache):
        if t.device != qkv.device:
            raise RuntimeError("all tensors must be on qkv's device")
    with _on_device(qkv.device):
        q_out = torch.empty((b, n_heads, s, head_dim), device=qkv.device, dtype=torch.bfloat16)
        _check(lib.astrai_w8a8_rope_cache_write_bf16(
            q2.data_ptr(), ld, freqs.contiguous().data_ptr(), positions.contiguous().data_ptr(),
            q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), b, s, n_heads, n_kv_heads,
            head_dim, k_cache.size(2), _stream(qkv)), lib)
    return q_out


def attn_decode_supported(n_heads: int, n_kv_heads: int, seq: int, head_dim: int) -> bool:
    """The shapes ``astrai_w8a8_attn_decode_bf16`` takes (the limits its entry point checks)."""
    return (head_dim == 128 and n_kv_heads > 0 and n_heads % n_kv_heads == 0
            and (n_heads // n_kv_heads) * seq <= 8 and n_heads <= 64)


def decode_nsplit(pairs: int, max_keys: int) -> int:
    """Context splits of the decode attention kernel for ``pairs`` (sequence, KV head) pairs whose
    contexts hold at most ``max_keys`` keys: up to 512 workgroups (two whole rounds of the 256
    compute units: 32 sequences x 4 KV heads run 4 splits, 1.352 ms a decode step, against 1.366 ms
    with 3 -- 1.5 workgroups per compute unit -- and 1.359 ms with 2), but no more than eight
    splits and no split shorter than ~160 keys of the longest possible context -- every split
    adds to the merge and to the launch (16 / 4 heads, 2 sequences x 520 keys: 11.7 us with 3
    splits against 15.5 us with 16; 32 x 520 keys: 18.9 us with 1)."""
    return max(1, min(8, 512 // max(1, pairs), max_keys // 160))


def attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, positions: torch.Tensor,
                scale: Optional[float] = None, nsplit: int = 0, quantized: bool = False):
    """``q [batch, n_heads, seq, 128]`` (bf16) against the dense caches
    ``[batch, n_kv_heads, max_len, 128]``; token ``s`` attends keys ``0..positions[s]``.
    Returns ``[batch, seq, n_heads * 128]`` bf16, or with ``quantized`` the per-token int8
    form of it ``(int8 [batch*seq, n_heads*128], fp32 [batch*seq, 1])``.
    ``nsplit`` 0 picks a split count that fills the chip."""
    lib = _require()
    _gpu(q, "attn_decode")
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("q and the caches must be bf16")
    if q.dim() != 4 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise RuntimeError("q must be [B, H, S, D] and the caches [B, H_kv, max_len, D]")
    b, h, s, d = q.shape
    hkv, max_len = k_cache.size(1), k_cache.size(2)
    if k_cache.size(0) != b or k_cache.size(3) != d:
        raise RuntimeError("cache batch / head_dim do not match q")
    if not (q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("q and the caches must be contiguous")
    if positions.dtype != torch.int64 or positions.numel() != s or positions.device != q.device:
        raise RuntimeError("positions must be int64 [seq] on q's device")
    if h % hkv:
        raise RuntimeError("n_heads must be a multiple of n_kv_heads")
    if scale is None:
        scale = d ** -0.5
    if nsplit <= 0:
        nsplit = decode_nsplit(b * hkv, max_len)
    nq = (h // hkv) * s
    with _on_device(q.device):
        need = lib.astrai_w8a8_attn_decode_workspace_floats(b, hkv, nsplit, nq)
        ws = torch.empty(max(need, 1), device=q.device, dtype=torch.float32)
        out = oq = os_ = None
        if quantized:
            oq = torch.empty((b * s, h * d), device=q.device, dtype=torch.int8)
            os_ = torch.empty((b * s, 1), device=q.device, dtype=torch.float32)
        else:
            out = torch.empty((b, s, h * d), device=q.device, dtype=torch.bfloat16)
        _check(lib.astrai_w8a8_attn_decode_bf16(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), positions.contiguous().data_ptr(),
            ws.data_ptr(), ws.numel(), _ptr(out), _ptr(oq), _ptr(os_), b, s, h, hkv, d, max_len, nsplit,
            float(scale), _stream(q)), lib)
    return (oq, os_) if quantized else out


STATIC_SCRATCH_FLOATS = 1 << 20


def attn_decode_static_scratch(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                               positions: torch.Tensor, out: Optional[torch.Tensor] = None,
                               out_q: Optional[torch.Tensor] = None, out_scale: Optional[torch.Tensor] = None,
                               scale: Optional[float] = None, nsplit: int = 1) -> None:
    """:func:`attn_decode` for callers that must not allocate: the caller brings the outputs
    (``out`` bf16 ``[batch, seq, n_heads*128]`` and / or ``out_q`` int8 with ``out_scale`` fp32
    ``[batch*seq]``), the context splits' partial results go to the array the library holds in
    static device memory (``STATIC_SCRATCH_FLOATS`` floats a GPU; larger requests are refused).
    Nothing is allocated here or in the library. Calls that overlap on one GPU share that
    array and race; calls ordered on one stream do not."""
    lib = _require()
    _gpu(q, "attn_decode_static_scratch")
    if q.dim() != 4 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise RuntimeError("q must be [B, H, S, D] and the caches [B, H_kv, max_len, D]")
    for t, dt, name in ((q, torch.bfloat16, "q"), (k_cache, torch.bfloat16, "k_cache"),
                        (v_cache, torch.bfloat16, "v_cache"), (positions, torch.int64, "positions"),
                        (out, torch.bfloat16, "out"), (out_q, torch.int8, "out_q"),
                        (out_scale, torch.float32, "out_scale")):
        if t is not None and (t.dtype != dt or not t.is_contiguous() or t.device != q.device):
            raise RuntimeError(f"{name} must be a contiguous {dt} tensor on q's device")
    b, h, s, d = q.shape
    hkv, max_len = k_cache.size(1), k_cache.size(2)
    if k_cache.size(0) != b or k_cache.size(3) != d or positions.numel() != s:
        raise RuntimeError("cache batch / head_dim or the number of positions do not match q")
    if (out is not None and out.numel() != b * s * h * d) or (out_q is not None and (
            out_q.numel() != b * s * h * d or out_scale is None or out_scale.numel() != b * s)):
        raise RuntimeError("out / out_q must hold batch*seq rows of n_heads*head_dim, out_scale batch*seq steps")
    with _on_device(q.device):
        _check(lib.astrai_w8a8_attn_decode_bf16_static_scratch(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), positions.data_ptr(), _ptr(out), _ptr(out_q),
            _ptr(out_scale), b, s, h, hkv, d, max_len, nsplit, float(d ** -0.5 if scale is None else scale),
            _stream(q)), lib)


def attn_paged_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                      kv_indptr: torch.Tensor, new_k: Optional[torch.Tensor] = None,
                      new_v: Optional[torch.Tensor] = None, mask: Optional[torch.Tensor] = None,
                      causal_offset: int = -1, scale: float = 0.0, o_part_buf=None, ml_part_buf=None,
                      out_buf: Optional[torch.Tensor] = None, nsplit: int = 0) -> torch.Tensor:
    """Paged decode attention with the argument list of the reference's pybind entry
    (csrc/kernels/attention/paged_decode.cu:69-86): ``q [batch, H, 128]``, flat pools
    ``[slots, H_kv, 128]``, ``req_to_token`` int32 ``[requests, max_context_len]``,
    ``req_pool_indices`` int32 ``[batch]``, ``kv_indptr`` int32 ``[batch+1]``; returns
    ``[batch, H, 128]`` bf16. ``new_k`` / ``new_v`` (``[batch, H_kv, 128]``) are first
    written to the slot of each sequence's newest position, as the reference's kernel
    persists them (layout_policies.cuh:226-252). ``causal_offset`` does not change a
    one-token query (layout_policies.cuh:194-197); ``o_part_buf`` (fp32, contiguous) serves as
    the split workspace when it is large enough, otherwise one is allocated here;
    ``ml_part_buf`` is not needed. ``mask``: bool ``[batch, width]``, True = attend
    that position (entry_utils.cuh:226-237); positions past ``width`` are not attended."""
    lib = _require()
    _gpu(q, "attn_paged_decode")
    if mask is not None:
        if not mask.is_cuda or mask.dtype != torch.bool:
            raise RuntimeError("mask must be bool CUDA")
        if mask.dim() != 2 or mask.size(0) != q.size(0):
            raise RuntimeError("mask batch mismatch: a decode mask is [batch, kv positions]")
        if mask.size(1) == 0:
            raise RuntimeError("mask kv_len mismatch: the mask has no positions")
        if mask.stride(1) != 1:
            mask = mask.contiguous()
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("q, k_cache and v_cache must be bf16")
    if q.dim() != 3 or k_cache.dim() != 3 or k_cache.shape != v_cache.shape:
        raise RuntimeError("q must be [batch, q_head, head_dim] and the pools [size, kv_head, head_dim]")
    for t, name in ((req_to_token, "req_to_token"), (req_pool_indices, "req_pool_indices"),
                    (kv_indptr, "kv_indptr")):
        if t.dtype != torch.int32 or t.device != q.device:
            raise RuntimeError(f"{name} must be int32 on q's device")
    b, h, d = q.shape
    slots, hkv = k_cache.size(0), k_cache.size(1)
    if k_cache.size(2) != d:
        raise RuntimeError("k_cache head_dim mismatch")
    if h % hkv:
        raise RuntimeError("q_head must be divisible by kv_head")
    if req_to_token.dim() != 2 or req_pool_indices.numel() != b or kv_indptr.numel() != b + 1:
        raise RuntimeError("req_to_token must be 2D, req_pool_indices [batch], kv_indptr [batch+1]")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("the pools must be contiguous")
    if (new_k is None) != (new_v is None):
        raise RuntimeError("new_k and new_v must be provided together")
    q_c = q.contiguous()
    rtt, rpi, ind = req_to_token.contiguous(), req_pool_indices.contiguous(), kv_indptr.contiguous()
    if scale is None or scale <= 0.0:
        scale = d ** -0.5
    user_nsplit = nsplit > 0
    if nsplit <= 0:
        nsplit = decode_nsplit(b * hkv, req_to_token.size(1))
    with _on_device(q.device):
        if new_k is not None:
            if new_k.shape != (b, hkv, d) or new_v.shape != (b, hkv, d):
                raise RuntimeError("new K/V shape mismatch")
            last = (ind[1:] - ind[:-1] - 1).long()
            dst = rtt[rpi.long(), last.clamp_min(0)].long()
            live = (last >= 0) & (dst >= 0)
            dst = torch.where(live, dst, torch.zeros_like(dst))
            # a sequence of length 0 has no newest position: it rewrites slot 0 with itself
            k_cache.index_put_((dst,), torch.where(live[:, None, None], new_k, k_cache[dst]))
            v_cache.index_put_((dst,), torch.where(live[:, None, None], new_v, v_cache[dst]))
        if out_buf is not None:
            if not (out_buf.is_cuda and out_buf.is_contiguous() and out_buf.dtype == q.dtype
                    and out_buf.dim() == 3 and out_buf.size(0) >= b and out_buf.shape[1:] == q.shape[1:]):
                raise RuntimeError("out_buf must be a contiguous [>=batch, q_head, head_dim] tensor of q's dtype")
            out = out_buf[:b]
        else:
            out = torch.empty((b, h, d), device=q.device, dtype=torch.bfloat16)
        if b == 0:
            return out  # (an empty tensor has no address to hand over)
        m_ptr, m_stride, m_width = (mask.data_ptr(), mask.stride(0), mask.size(1)) if mask is not None else (0, 0, 0)
        if d != 128 or h > 64 or h // hkv > 8:  # the shapes only the general kernel takes
            if not user_nsplit:  # one wave per (sequence, kv head, split): enough of them to fill the chip
                nsplit = max(1, min(64, 2048 // max(1, b * hkv), rtt.size(1) // 64))
            _paged_rows(lib, q_c, k_cache, v_cache, rtt, rpi, ind, None, (m_ptr, m_stride, 0, 0, 1, m_width),
                        out, b, nsplit, False, scale, o_part_buf)
            return out
        need = lib.astrai_w8a8_attn_decode_workspace_floats(b, hkv, nsplit, h // hkv)
        ws = _scratch(need, q.device, o_part_buf)
        _check(lib.astrai_w8a8_attn_paged_decode_masked_bf16(
            q_c.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), rtt.data_ptr(), rpi.data_ptr(),
            ind.data_ptr(), m_ptr, m_stride, m_width, ws.data_ptr(), ws.numel(), out.data_ptr(), b, h, hkv,
            d, slots, rtt.size(0), rtt.size(1), nsplit, float(scale), _stream(q)), lib)
    return out


def _scratch(need: int, device, given: Optional[torch.Tensor]) -> torch.Tensor:
    """``need`` fp32 elements of scratch: the caller's pre-allocated buffer when it is large
    enough (the reference's callers hand over their split buffers so that a captured decode step
    allocates nothing), else a fresh tensor."""
    if given is not None and given.is_cuda and given.device == device and given.dtype == torch.float32 \
            and given.is_contiguous() and given.numel() >= need:
        return given.view(-1)
    return torch.empty(max(need, 1), device=device, dtype=torch.float32)


def _paged_rows(lib, q, k_pool, v_pool, rtt, rpi, kv_indptr, schedule, m_args, out, count, nsplit, causal,
                scale, scratch: Optional[torch.Tensor] = None) -> None:
    """The general paged kernel (any head_dim in {32, 64, 128, 256}, n_rep <= 8). ``schedule``:
    ``(qo_indptr, q_tile_to_batch, q_tile_to_index)`` for a prefill call (``count`` = tiles),
    None for decode (``count`` = batch)."""
    h, d, hkv = q.size(1), q.size(2), k_pool.size(1)
    prefill = schedule is not None
    need = lib.astrai_w8a8_attn_paged_rows_workspace_floats(count, h, hkv, d, nsplit, 1 if prefill else 0)
    if need < 0:
        raise RuntimeError(f"paged attention needs head_dim in (32, 64, 128, 256) and n_heads / n_kv_heads <= 16; "
                           f"got head_dim {d}, {h} / {hkv} heads")
    ws = _scratch(need, q.device, scratch)
    sched = [t.data_ptr() for t in schedule] if prefill else [0, 0, 0]
    _check(lib.astrai_w8a8_attn_paged_rows_bf16(
        q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), rtt.data_ptr(), rpi.data_ptr(), kv_indptr.data_ptr(),
        *sched, *m_args, ws.data_ptr(), ws.numel(), out.data_ptr(), count, h, hkv, d, k_pool.size(0), rtt.size(0),
        rtt.size(1), 1 if causal else 0, nsplit, float(scale), _stream(q)), lib)


Q_TILE_ROWS = 64  # rows per tile of the schedule the reference builds (astrai/inference/workspace.py:13)


def attn_paged_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                       kv_indptr: torch.Tensor, qo_indptr: torch.Tensor,
                       q_tile_to_batch: torch.Tensor, q_tile_to_index: torch.Tensor,
                       mask: Optional[torch.Tensor] = None, causal_offset: int = -1,
                       scale: float = 0.0, nsplit: int = 0) -> torch.Tensor:
    """Ragged paged prefill with the argument list of the reference's pybind entry
    (csrc/kernels/attention/paged_prefill.cu:36-52): packed ``q [total_q, H, 128]``, flat
    pools, ``req_to_token`` / ``req_pool_indices`` / ``kv_indptr`` / ``qo_indptr`` int32, and
    the schedule of 64-row query tiles. ``causal_offset >= 0`` asks for the causal mask (the
    wrapper passes 0 for ``is_causal``, astrai/extension/ops/attention.py:188). ``mask``:
    bool, True = attend, ``[batch, kv]`` or ``[batch, 1 | H, rows, kv]`` with ``rows`` counted
    inside each sequence (entry_utils.cuh:326-346); rows and positions the mask does not hold
    are not attended. Returns ``[total_q, H, head_dim]`` bf16. head_dim 128 with a grouping of
    2, 4 or 8 runs the MFMA block kernel; other shapes the general kernel, whose context split
    ``nsplit`` (0: chosen here) only matters for short schedules."""
    lib = _require()
    _gpu(q, "attn_paged_prefill")
    m_args = (0, 0, 0, 0, 0, 0)
    if mask is not None:
        if not mask.is_cuda or mask.dtype != torch.bool:
            raise RuntimeError("mask must be bool CUDA")
        if mask.dim() not in (2, 4):
            raise RuntimeError("mask must be 2D or 4D")
        if mask.size(0) != req_pool_indices.numel():
            raise RuntimeError("mask batch mismatch")
        if mask.dim() == 4 and mask.size(1) not in (1, q.size(1)):
            raise RuntimeError("mask head mismatch")
        if mask.dim() == 4 and mask.size(2) == 0:
            raise RuntimeError("mask q_len mismatch")
        if mask.size(-1) == 0:
            raise RuntimeError("mask kv_len mismatch: the mask has no positions")
        if mask.stride(-1) != 1:
            mask = mask.contiguous()
        if mask.dim() == 2:
            m_args = (mask.data_ptr(), mask.stride(0), 0, 0, 1, mask.size(1))
        else:
            m_args = (mask.data_ptr(), mask.stride(0), 0 if mask.size(1) == 1 else mask.stride(1),
                      0 if mask.size(2) == 1 else mask.stride(2), mask.size(2), mask.size(3))
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("q, k_cache and v_cache must be bf16")
    if q.dim() != 3 or k_cache.dim() != 3 or k_cache.shape != v_cache.shape:
        raise RuntimeError("q must be [total_q, q_head, head_dim] and the pools [size, kv_head, head_dim]")
    ints = ((req_to_token, "req_to_token"), (req_pool_indices, "req_pool_indices"), (kv_indptr, "kv_indptr"),
            (qo_indptr, "qo_indptr"), (q_tile_to_batch, "q_tile_to_batch"), (q_tile_to_index, "q_tile_to_index"))
    for t, name in ints:
        if t.dtype != torch.int32 or t.device != q.device:
            raise RuntimeError(f"{name} must be int32 on q's device")
    total_q, h, d = q.shape
    slots, hkv = k_cache.size(0), k_cache.size(1)
    b = req_pool_indices.numel()
    if k_cache.size(2) != d:
        raise RuntimeError("k_cache head_dim mismatch")
    if h % hkv:
        raise RuntimeError("q_head must be divisible by kv_head")
    if req_to_token.dim() != 2 or kv_indptr.numel() != b + 1 or qo_indptr.numel() != b + 1:
        raise RuntimeError("req_to_token must be 2D, kv_indptr and qo_indptr [batch+1]")
    if q_tile_to_batch.dim() != 1 or q_tile_to_batch.shape != q_tile_to_index.shape:
        raise RuntimeError("q_tile_to_batch and q_tile_to_index must be 1D of equal length")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("the pools must be contiguous")
    q_c = q.contiguous()
    tensors = [t.contiguous() for t, _ in ints]
    if scale is None or scale <= 0.0:
        scale = d ** -0.5
    with _on_device(q.device):
        # (rows that no tile of the schedule covers are left unwritten, as by the reference)
        out = torch.empty((total_q, h, d), device=q.device, dtype=torch.bfloat16)
        if total_q == 0 or q_tile_to_batch.numel() == 0:
            return out  # (an empty tensor has no address to hand over)
        if not attn_prefill_supported(h, hkv, d):  # the shapes only the general kernel takes
            tiles = q_tile_to_batch.numel()
            waves = tiles * 4 * hkv                  # at least: one wave per row block, 4+ blocks per tile
            _paged_rows(lib, q_c, k_cache, v_cache, tensors[0], tensors[1], tensors[2], tensors[3:], m_args,
                        out, tiles, nsplit if nsplit > 0 else max(1, min(16, 2048 // max(1, waves))),
                        causal_offset >= 0, scale)
            return out
        _check(lib.astrai_w8a8_attn_paged_prefill_masked_bf16(
            q_c.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), *[t.data_ptr() for t in tensors],
            *m_args, out.data_ptr(), q_tile_to_batch.numel(), h, hkv, d, slots, req_to_token.size(0),
            req_to_token.size(1), 1 if causal_offset >= 0 else 0, float(scale), _stream(q)), lib)
    return out


def paged_prefill_schedule(q_lens, device):
    """``(qo_indptr, q_tile_to_batch, q_tile_to_index)`` for per-sequence query row counts,
    built as astrai/inference/cache/pool.py:219-234 builds them (64-row tiles)."""
    qo = [0]
    tb, ti = [], []
    for i, n in enumerate(q_lens):
        qo.append(qo[-1] + int(n))
        nt = (int(n) + Q_TILE_ROWS - 1) // Q_TILE_ROWS
        tb += [i] * nt
        ti += list(range(nt))
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return mk(qo), mk(tb), mk(ti)


def attn_prefill_supported(n_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    return head_dim == 128 and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads in (2, 4, 8)


def attn_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 positions: torch.Tensor, scale: Optional[float] = None) -> torch.Tensor:
    """Causal attention of ``q [batch, n_heads, seq, 128]`` (bf16) against the dense caches
    ``[batch, n_kv_heads, max_len, 128]``; token ``s`` attends keys ``0..positions[s]``.
    Returns ``[batch, seq, n_heads * 128]`` bf16 (token-major, what ``o_proj`` reads)."""
    lib = _require()
    _gpu(q, "attn_prefill")
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("q and the caches must be bf16")
    if q.dim() != 4 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise RuntimeError("q must be [B, H, S, D] and the caches [B, H_kv, max_len, D]")
    b, h, s, d = q.shape
    hkv, max_len = k_cache.size(1), k_cache.size(2)
    if k_cache.size(0) != b or k_cache.size(3) != d:
        raise RuntimeError("cache batch / head_dim do not match q")
    if not (q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("q and the caches must be contiguous")
    if positions.dtype != torch.int64 or positions.numel() != s or positions.device != q.device:
        raise RuntimeError("positions must be int64 [seq] on q's device")
    if h % hkv:
        raise RuntimeError("n_heads must be a multiple of n_kv_heads")
    if scale is None:
        scale = d ** -0.5
    with _on_device(q.device):
        out = torch.empty((b, s, h * d), device=q.device, dtype=torch.bfloat16)
        _check(lib.astrai_w8a8_attn_prefill_bf16(
            q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), positions.contiguous().data_ptr(),
            out.data_ptr(), b, s, h, hkv, d, max_len, float(scale), _stream(q)), lib)
    return out


_INT8_ENTRY = {
    "auto": "astrai_w8a8_gemm_int8_ptpc",
    "gemv": "astrai_w8a8_gemv_int8_ptpc",
    "tiled": "astrai_w8a8_gemm_int8_ptpc_tiled",
}


def _int8_operands(a, b, sa, sb, bias, need_scales: bool, what: str):
    """The checks every int8 NT GEMM wrapper makes on its operands; returns contiguous operands
    (K zero-padded where ``_pad_k`` says so), checked scale vectors and bias, and ``(m, n, k)``
    with the K to hand to the library."""
    _gpu(a, what)
    _gpu(b, what)
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise RuntimeError("a and b must be int8")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("a and b must be 2D")
    if a.device != b.device:
        raise RuntimeError("a and b must be on the same device")
    if a.size(1) != b.size(1):
        raise RuntimeError("inner dim mismatch")
    a_c, b_c = a.contiguous(), b.contiguous()
    m, k = a_c.shape
    n = b_c.size(0)
    if need_scales:
        if sa is None or sb is None:
            raise RuntimeError("bf16 output requires sa and sb")
        sa = _check_vec(sa, a, m, "sa")
        sb = _check_vec(sb, a, n, "sb")
    if bias is not None:
        if not (bias.is_cuda and bias.device == a.device and bias.dtype == torch.bfloat16
                and bias.numel() == n):
            raise RuntimeError("bias must be CUDA bf16 with shape [N]")
        bias = bias.contiguous()
    with _on_device(a.device):
        a_c, b_c, k = _pad_k(a_c, b_c)
    return a_c, b_c, sa, sb, bias, m, n, k


def mm_int8(a: torch.Tensor, b: torch.Tensor, sa: Optional[torch.Tensor],
            sb: Optional[torch.Tensor], bias: Optional[torch.Tensor] = None,
            out_dtype: int = 0, kernel: str = "auto") -> torch.Tensor:
    """int8 NT GEMM. ``out_dtype`` 0: ``bf16(acc*sa[m]*sb[n] (+bias))``; 2: raw int32
    accumulator. ``kernel`` names the entry point: auto / gemv / tiled."""
    lib = _require()
    if out_dtype not in (OUT_BF16, OUT_ACC):
        raise RuntimeError("out_dtype must be 0 (bf16) or 2 (int32 accumulator)")
    a_c, b_c, sa, sb, bias, m, n, k = _int8_operands(a, b, sa, sb, bias, out_dtype == OUT_BF16, "mm_int8")
    fn = getattr(lib, _INT8_ENTRY[kernel])
    with _on_device(a.device):
        out = torch.empty((m, n), device=a.device,
                          dtype=torch.int32 if out_dtype == OUT_ACC else torch.bfloat16)
        if m and n:
            if k == 0:
                out.zero_()
            else:
                _check(fn(a_c.data_ptr(), b_c.data_ptr(), _ptr(sa), _ptr(sb), _ptr(bias),
                          out.data_ptr(), m, n, k, out_dtype, _stream(a)), lib)
    return out


def mm_int8_resid(a: torch.Tensor, b: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor,
                  resid: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``mm_int8(a, b, sa, sb, bias) + resid`` in bf16 arithmetic, the addition done in the
    GEMM's epilogue where the shape has one (``attn_output + x`` / ``mlp_output + x`` of
    astrai/model/components/decoder_block.py:67,70). ``resid`` bf16 ``[M, N]``; returns a new
    bf16 ``[M, N]`` tensor, bit for bit the two separate operations."""
    lib = _require()
    a_c, b_c, sa, sb, bias, m, n, k = _int8_operands(a, b, sa, sb, bias, True, "mm_int8_resid")
    if not (resid.is_cuda and resid.device == a.device and resid.dtype == torch.bfloat16
            and resid.numel() == m * n):
        raise RuntimeError("resid must be CUDA bf16 with M*N elements")
    resid_c = resid.contiguous()
    with _on_device(a.device):
        out = torch.empty((m, n), device=a.device, dtype=torch.bfloat16)
        if m and n:
            if k == 0:
                out.copy_(resid_c.reshape(m, n) if bias is None
                          else (bias.reshape(1, n).expand(m, n) + resid_c.reshape(m, n)))
            else:
                _check(lib.astrai_w8a8_gemm_int8_ptpc_resid(
                    a_c.data_ptr(), b_c.data_ptr(), _ptr(sa), _ptr(sb), _ptr(bias), resid_c.data_ptr(),
                    out.data_ptr(), m, n, k, _stream(a)), lib)
    return out


def last_kernel() -> str:
    """Family name of the kernel the most recent GEMM entry of this thread launched
    (diagnostic; ``astrai_w8a8_last_kernel``)."""
    return _require().astrai_w8a8_last_kernel().decode()


def mfma_probe(kind: int, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """One MFMA of shape ``kind`` on a zero accumulator in one wave (test hook); returns the
    raw accumulator registers ``[64, 4]`` or ``[64, 16]`` as int32 words."""
    lib = _require()
    _gpu(a, "mfma_probe")
    rows, kbytes = {0: (16, 64), 1: (16, 128), 2: (16, 128), 3: (32, 32), 4: (32, 64), 5: (32, 64),
                    6: (16, 64), 7: (32, 32)}[kind]
    for t in (a, b):
        if not t.is_contiguous() or t.numel() * t.element_size() != rows * kbytes or t.device != a.device:
            raise RuntimeError(f"operands of kind {kind} are contiguous [{rows}] rows of {kbytes} bytes")
    with _on_device(a.device):
        d = torch.zeros((64, 4 if rows == 16 else 16), device=a.device, dtype=torch.int32)
        _check(lib.astrai_w8a8_mfma_probe(kind, a.data_ptr(), b.data_ptr(), d.data_ptr(), _stream(a)), lib)
    return d


SWIGLU_BLOCK = 64


def swiglu_block_rows(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of ``gate`` and ``up`` (``[W, ...]`` each, W a multiple of 64) in the order the
    SwiGLU GEMM entry points take: blocks of 128 rows, 64 of gate then the 64 of up that
    belong to the same columns of ``h``."""
    w = gate.size(0)
    if up.shape != gate.shape or w % SWIGLU_BLOCK:
        raise RuntimeError("gate and up must have the same shape with a multiple of 64 rows")
    rest = gate.shape[1:]
    g = gate.reshape(w // SWIGLU_BLOCK, 1, SWIGLU_BLOCK, *rest)
    u = up.reshape(w // SWIGLU_BLOCK, 1, SWIGLU_BLOCK, *rest)
    return torch.cat((g, u), dim=1).reshape(2 * w, *rest).contiguous()


def mm_int8_swiglu_fused_shape(m: int, n: int, k: int) -> bool:
    """Shapes whose gate|up GEMM applies the SwiGLU product in its own epilogue (the limits
    of ``astrai_w8a8_gemm_int8_ptpc_swiglu``); others run the GEMM and the blocked producer."""
    tiles = ((m + 255) // 256) * ((n + 255) // 256)
    return (tiles >= 192 and k >= 256 and k % 128 == 0 and n % 128 == 0 and n <= 1 << 22
            and m * k < 2 ** 31 and n * k < 2 ** 31 and n // 2 <= FUSED_ROW_MAX)


def mm_int8_swiglu(a: torch.Tensor, wgu: torch.Tensor, sa: torch.Tensor, sgu: torch.Tensor,
                   want_h: bool = False, fused: Optional[bool] = None):
    """``h = up * silu(gate)`` of the gate and up projections of ``a`` and its per-row int8
    form, ``wgu`` / ``sgu`` being the int8 weight and its scales in :func:`swiglu_block_rows`
    order. Returns ``(hq [M, W], s [M, 1], h or None)``, bit for bit what :func:`mm_int8` on
    the unblocked weight followed by :func:`silu_mul_quantize_int8` gives. Large shapes run
    the GEMM whose epilogue forms ``h`` and the row maxima piecewise, then the one-read
    quantizer; others the plain GEMM and the producer that reads the blocked columns
    (``fused`` forces one or the other)."""
    lib = _require()
    _gpu(a, "mm_int8_swiglu")
    if a.dtype != torch.int8 or wgu.dtype != torch.int8 or a.dim() != 2 or wgu.dim() != 2:
        raise RuntimeError("a and wgu must be 2D int8")
    if a.size(1) != wgu.size(1) or a.device != wgu.device:
        raise RuntimeError("inner dim or device mismatch")
    m, k = a.shape
    n = wgu.size(0)
    if n % (2 * SWIGLU_BLOCK):
        raise RuntimeError("wgu must hold blocks of 64 gate and 64 up rows")
    w = n // 2
    if not fused_rows_supported(w):
        raise RuntimeError(f"h rows of {w} columns are outside what the quantizer takes")
    if fused is None:
        fused = mm_int8_swiglu_fused_shape(m, n, k)
    if not fused:
        gu = mm_int8(a, wgu, sa, sgu)
        with _on_device(a.device):
            hq = torch.empty((m, w), device=a.device, dtype=torch.int8)
            s = torch.empty((m, 1), device=a.device, dtype=torch.float32)
            h = torch.empty((m, w), device=a.device, dtype=torch.bfloat16) if want_h else None
            if m:
                _check(lib.astrai_w8a8_silu_mul_quantize_int8_rows_blocked(
                    gu.data_ptr(), n, SWIGLU_BLOCK, _ptr(h), hq.data_ptr(), s.data_ptr(), m, w,
                    _stream(a)), lib)
        return hq, s, h
    a_c, w_c = a.contiguous(), wgu.contiguous()
    sa = _check_vec(sa, a, m, "sa")
    sgu = _check_vec(sgu, a, n, "sgu")
    pieces = n // 128
    with _on_device(a.device):
        h = torch.empty((m, w), device=a.device, dtype=torch.bfloat16)
        row_max = torch.empty((m, pieces), device=a.device, dtype=torch.float32)
        hq = torch.empty((m, w), device=a.device, dtype=torch.int8)
        s = torch.empty((m, 1), device=a.device, dtype=torch.float32)
        _check(lib.astrai_w8a8_gemm_int8_ptpc_swiglu(
            a_c.data_ptr(), w_c.data_ptr(), sa.data_ptr(), sgu.data_ptr(), h.data_ptr(),
            row_max.data_ptr(), m, n, k, _stream(a)), lib)
        _check(lib.astrai_w8a8_quantize_int8_rows_pmax(
            h.data_ptr(), row_max.data_ptr(), pieces, hq.data_ptr(), s.data_ptr(), m, w,
            _stream(a)), lib)
    return hq, s, (h if want_h else None)


def mm_int8_rope_cache_supported(tokens: int, k: int, head_dim: int, n: int = 0, batch: int = 0,
                                 n_heads: int = 0, n_kv_heads: int = 0, max_len: int = 0) -> bool:
    """Shapes the fused q|k|v projection + rotary + cache-write entry takes (the limits it
    checks); ``n`` = rows of the q|k|v weight, when known. A few tokens (decode steps: at most
    64, K % 256 == 0, head_dim % 4 == 0) run the row-range kernel; long blocks (prefill: head_dim
    128, at least 192 output tiles of 256 x 256, K % 128 == 0, destinations under 2 GiB -- checked
    when ``batch`` .. ``max_len`` are given) the large-tile GEMM with the same epilogue."""
    if tokens <= 0 or n * k >= 2 ** 31 or tokens * k >= 2 ** 31:
        return False
    if tokens <= 64 and k % 256 == 0 and head_dim % 4 == 0:
        return True
    tiles = ((tokens + 255) // 256) * ((n + 255) // 256)
    return (head_dim == 128 and n > 0 and n % 128 == 0 and tiles >= 192 and k >= 256 and k % 128 == 0
            and tokens * n_heads * 256 < 2 ** 31 and batch * n_kv_heads * max_len * 256 < 2 ** 31)


FUSED_ROW_MAX = 8192


def fused_rows_supported(width: int) -> bool:
    """Row widths the producers fused with the per-token quantizer take
    (``add_rmsnorm_quantize_int8_rows``, ``silu_mul_quantize_int8_rows``)."""
    return width % 8 == 0 and 0 <= width <= FUSED_ROW_MAX


def mm_int8_rope_cache(a: torch.Tensor, wqkv: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor,
                       freqs: torch.Tensor, positions: torch.Tensor, k_cache: torch.Tensor,
                       v_cache: torch.Tensor, batch: int, seq: int, n_heads: int, n_kv_heads: int,
                       head_dim: int) -> torch.Tensor:
    """``mm_int8(a, wqkv, sa, sb)`` followed by :func:`rope_cache_write` on its output, as one
    kernel and bit for bit the same: ``a`` int8 ``[batch*seq, K]`` (a few rows or a long block, see
    :func:`mm_int8_rope_cache_supported`), ``wqkv``
    int8 ``[(n_heads + 2 n_kv_heads) * head_dim, K]``. Writes k and v into the caches at
    ``positions`` and returns the rotated q as ``[batch, n_heads, seq, head_dim]``."""
    lib = _require()
    _gpu(a, "mm_int8_rope_cache")
    if a.dtype != torch.int8 or wqkv.dtype != torch.int8 or a.dim() != 2 or wqkv.dim() != 2:
        raise RuntimeError("a and wqkv must be 2D int8")
    m, k = a.shape
    n = (n_heads + 2 * n_kv_heads) * head_dim
    if m != batch * seq or wqkv.size(0) != n or wqkv.size(1) != k:
        raise RuntimeError("a must be [batch*seq, K] and wqkv [(n_heads + 2 n_kv_heads) * head_dim, K]")
    if not mm_int8_rope_cache_supported(m, k, head_dim, n, batch, n_heads, n_kv_heads, k_cache.size(2)):
        raise RuntimeError("mm_int8_rope_cache: needs at most 64 tokens with K % 256 == 0 and head_dim % 4 == 0, "
                           "or head_dim 128 with at least 192 output tiles of 256 x 256 and K % 128 == 0; "
                           "operands and destinations under 2 GiB")
    sa = _check_vec(sa, a, m, "sa")
    sb = _check_vec(sb, a, n, "sb")
    if k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise RuntimeError("the caches must be bf16")
    if freqs.dtype != torch.float32 or tuple(freqs.shape[-3:]) != (seq, head_dim // 2, 2):
        raise RuntimeError("freqs must be fp32 [seq, head_dim/2, 2]")
    if positions.dtype != torch.int64 or positions.numel() != seq:
        raise RuntimeError("positions must be int64 [seq]")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()) or k_cache.shape != v_cache.shape:
        raise RuntimeError("caches must be contiguous and of one shape")
    if k_cache.dim() != 4 or k_cache.size(0) != batch or k_cache.size(1) != n_kv_heads or k_cache.size(3) != head_dim:
        raise RuntimeError("caches must be [batch, n_kv_heads, max_len, head_dim]")
    for t in (wqkv, freqs, positions, k_cache, v_cache):
        if t.device != a.device:
            raise RuntimeError("all tensors must be on a's device")
    a_c, w_c = a.contiguous(), wqkv.contiguous()
    with _on_device(a.device):
        q_out = torch.empty((batch, n_heads, seq, head_dim), device=a.device, dtype=torch.bfloat16)
        _check(lib.astrai_w8a8_gemm_int8_ptpc_rope_cache(
            a_c.data_ptr(), w_c.data_ptr(), sa.data_ptr(), sb.data_ptr(), freqs.contiguous().data_ptr(),
            positions.contiguous().data_ptr(), q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
            batch, seq, n_heads, n_kv_heads, head_dim, k_cache.size(2), k, _stream(a)), lib)
    return q_out


def quantize_fp8_block128_act(x: torch.Tensor):
    """bf16 ``[M,K]`` -> ``(x8 e4m3fn [M,K], sa fp32 [M,K/128])``."""
    lib = _require()
    _gpu(x, "quantize_fp8_block128_act")
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise RuntimeError("x must be 2D bf16")
    m, k = x.shape
    if k % 128:
        raise RuntimeError("K must be a multiple of 128")
    x_c = x.contiguous()
    with _on_device(x.device):
        x8 = torch.empty((m, k), device=x.device, dtype=torch.float8_e4m3fn)
        sa = torch.empty((m, k // 128), device=x.device, dtype=torch.float32)
        if m and k:
            _check(lib.astrai_w8a8_quantize_bf16_fp8_block128_act(
                x_c.data_ptr(), x8.data_ptr(), sa.data_ptr(), m, k, _stream(x)), lib)
    return x8, sa


def quantize_fp8_block128_weight(w: torch.Tensor):
    """bf16 ``[N,K]`` -> ``(w8 e4m3fn [N,K], sb fp32 [ceil(N/128),K/128])``."""
    lib = _require()
    _gpu(w, "quantize_fp8_block128_weight")
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise RuntimeError("w must be 2D bf16")
    n, k = w.shape
    if k % 128:
        raise RuntimeError("K must be a multiple of 128")
    w_c = w.contiguous()
    with _on_device(w.device):
        w8 = torch.empty((n, k), device=w.device, dtype=torch.float8_e4m3fn)
        sb = torch.empty(((n + 127) // 128, k // 128), device=w.device, dtype=torch.float32)
        if n and k:
            _check(lib.astrai_w8a8_quantize_bf16_fp8_block128_weight(
                w_c.data_ptr(), w8.data_ptr(), sb.data_ptr(), n, k, _stream(w)), lib)
    return w8, sb


def mm_fp8_block128(a: torch.Tensor, b: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor,
                    bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """e4m3fn NT GEMM with ``sa [M,K/128]`` and ``sb [ceil(N/128),K/128]`` block scales."""
    lib = _require()
    _gpu(a, "mm_fp8_block128")
    _gpu(b, "mm_fp8_block128")
    if a.dtype != torch.float8_e4m3fn or b.dtype != torch.float8_e4m3fn:
        raise RuntimeError("a and b must be fp8 e4m3fn")
    if a.dim() != 2 or b.dim() != 2 or a.size(1) != b.size(1):
        raise RuntimeError("a and b must be 2D with matching inner dim")
    if a.device != b.device:
        raise RuntimeError("a and b must be on the same device")
    a_c, b_c = a.contiguous(), b.contiguous()
    m, k = a_c.shape
    n = b_c.size(0)
    if k % 128 or k == 0:
        raise RuntimeError("K must be a positive multiple of 128")
    kb = k // 128
    sa = _check_vec(sa, a, m * kb, "sa")
    sb = _check_vec(sb, a, ((n + 127) // 128) * kb, "sb")
    if bias is not None:
        if not (bias.is_cuda and bias.device == a.device and bias.dtype == torch.bfloat16
                and bias.numel() == n):
            raise RuntimeError("bias must be CUDA bf16 with shape [N]")
        bias = bias.contiguous()
    with _on_device(a.device):
        out = torch.empty((m, n), device=a.device, dtype=torch.bfloat16)
        if m and n:
            _check(lib.astrai_w8a8_gemm_fp8_block128(
                a_c.data_ptr(), b_c.data_ptr(), sa.data_ptr(), sb.data_ptr(), _ptr(bias),
                out.data_ptr(), m, n, k, _stream(a)), lib)
    return out


# ---------------------------------------------------------------------------
# The reference's dense entries attn_decode / attn_prefill (q, k, v tensors in either
# layout, csrc/kernels/attention/decode.cu:4-67 and prefill.cu) on top of the kernels above.
# ---------------------------------------------------------------------------

BHLD, BLHD = 0, 1  # the reference's TensorLayout (csrc/kernels/attention/common.h)

_index_cache: dict = {}


def _identity_paging(batch: int, kv_len: int, device):
    """``(req_to_token, req_pool_indices)`` that address a token-major ``[batch, kv_len, ...]``
    tensor, viewed as a pool of ``batch * kv_len`` slots, sequence by sequence."""
    key = ("page", batch, kv_len, str(device))
    if key not in _index_cache:
        if len(_index_cache) > 64:
            _index_cache.clear()
        table = torch.arange(batch * kv_len, dtype=torch.int32, device=device).reshape(batch, kv_len)
        _index_cache[key] = (table, torch.arange(batch, dtype=torch.int32, device=device))
    return _index_cache[key]


def _dense_args(q, k, v, layout, what):
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError(f"{what}: q, k and v must be CUDA tensors")
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise RuntimeError(f"{what}: q, k and v must be bf16")
    if k.shape != v.shape:
        raise RuntimeError("K and V must have identical shapes")
    if q.dim() != 4 or k.dim() != 4:
        raise RuntimeError("Q/K/V must be 4D")
    if layout not in (BHLD, BLHD):
        raise RuntimeError(f"{what}: layout must be 0 (BHLD) or 1 (BLHD)")
    l_ax, h_ax = (2, 1) if layout == BHLD else (1, 2)
    b, q_len, h, d = q.size(0), q.size(l_ax), q.size(h_ax), q.size(3)
    kv_len, hkv = k.size(l_ax), k.size(h_ax)
    if k.size(0) != b:
        raise RuntimeError("K/V batch must match Q")
    if h % hkv:
        raise RuntimeError("q_head must be divisible by kv_head")
    if k.size(3) != d:
        raise RuntimeError("K/V head_dim must match Q")
    return b, q_len, kv_len, h, hkv, d


def _dense_mask(mask, b, q_len, kv_len, h):
    """The reference's 2D / 3D / 4D mask (entry_utils.cuh:56-86) as ``[b, 1 | h, 1 | q_len, kv_len]``."""
    if mask is None:
        return None
    if not mask.is_cuda:
        raise RuntimeError("mask must be on CUDA")
    if mask.dtype != torch.bool:
        raise RuntimeError("mask must be bool")
    if mask.size(0) != b:
        raise RuntimeError("mask batch mismatch")
    if mask.size(-1) != kv_len:
        raise RuntimeError("mask kv_len mismatch")
    if mask.dim() == 2:
        return mask[:, None, None, :]
    if mask.dim() == 3:
        if mask.size(1) not in (1, q_len):
            raise RuntimeError("mask q_len mismatch")
        return mask[:, None]
    if mask.dim() == 4:
        if mask.size(1) not in (1, h):
            raise RuntimeError("mask head mismatch")
        if mask.size(2) not in (1, q_len):
            raise RuntimeError("mask q_len mismatch")
        return mask
    raise RuntimeError("mask must be 2D, 3D, or 4D")


def _token_major(t, layout):
    return (t.transpose(1, 2) if layout == BHLD else t).contiguous()


def attn_cache_rows_supported(n_heads: int, n_kv_heads: int, head_dim: int) -> bool:
    """Head shapes :func:`attn_cache_rows` takes (those of the general paged kernel)."""
    return head_dim in (32, 64, 128, 256) and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16


def cache_context_len(positions: torch.Tensor, max_len: int) -> torch.Tensor:
    """Number of cache positions a block of new tokens at ``positions`` can attend to: newest
    position + 1, never more than the cache holds (rotary / cache-write kernels skip positions
    at or past ``max_len``, so a model that runs past its cache must not read past it either).
    An int32 scalar on ``positions``' device; nothing is read on the host."""
    return torch.clamp(positions.max() + 1, min=0, max=max_len).to(torch.int32)


def attn_cache_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    positions: torch.Tensor) -> torch.Tensor:
    """Attention of new tokens ``q [batch, n_heads, seq, head_dim]`` at ``positions [seq]``
    (int64, on the device) against the dense head-major caches ``[batch, n_kv_heads, max_len,
    head_dim]`` through the general paged kernel, for the head shapes the tuned dense kernels
    do not take (head_dim 32 / 64 / 256, any grouping up to 16). Every (sequence, KV head) pair
    is addressed as one sequence of a one-head pool -- the cache rows of a KV head are
    contiguous -- with the pair's query heads as its heads; nothing of the cache is copied
    and no length is read on the host. A row attends keys at positions <= its own. Returns
    token-major ``[batch, seq, n_heads * head_dim]``."""
    _gpu(q, "attn_cache_rows")
    b, h, s, d = q.shape
    hkv, max_len = k_cache.size(1), k_cache.size(2)
    if not attn_cache_rows_supported(h, hkv, d):
        raise RuntimeError(f"attn_cache_rows: head_dim {d} with {h} / {hkv} heads is not supported")
    if k_cache.shape != (b, hkv, max_len, d) or v_cache.shape != k_cache.shape \
            or not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise RuntimeError("attn_cache_rows: the caches must be contiguous [batch, n_kv_heads, max_len, head_dim]")
    n_rep, pairs = h // hkv, b * hkv
    with _on_device(q.device):
        table, rows = _identity_paging(pairs, max_len, q.device)
        key = ("ramp", pairs, str(q.device))
        if key not in _index_cache:
            _index_cache[key] = torch.arange(pairs + 1, dtype=torch.int32, device=q.device)
        kv_indptr = _index_cache[key] * cache_context_len(positions, max_len)
        k_pool, v_pool = k_cache.view(pairs * max_len, 1, d), v_cache.view(pairs * max_len, 1, d)
        if s == 1:
            out = attn_paged_decode(q.reshape(pairs, n_rep, d), k_pool, v_pool, table, rows, kv_indptr)
            return out.reshape(b, 1, h * d)
        key = ("sched", pairs, s, str(q.device))
        if key not in _index_cache:
            _index_cache[key] = paged_prefill_schedule([s] * pairs, q.device)
        qo, tb, ti = _index_cache[key]
        # rows of a pair token-major: [pair, seq, n_rep, head_dim]
        q_tm = q.reshape(b, hkv, n_rep, s, d).transpose(2, 3).reshape(pairs * s, n_rep, d)
        mask = (torch.arange(max_len, device=q.device)[None, :] <= positions[:, None])  # [seq, max_len]
        out = attn_paged_prefill(q_tm, k_pool, v_pool, table, rows, kv_indptr, qo, tb, ti,
                                 mask=mask[None, None].expand(pairs, 1, s, max_len))
    return out.view(b, hkv, s, n_rep, d).permute(0, 2, 1, 3, 4).reshape(b, s, h * d)


def attn_decode_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor] = None,
                    causal_offset: int = -1, scale: float = 0.0, layout: int = BHLD,
                    o_part_buf=None, ml_part_buf=None) -> torch.Tensor:
    """The reference's ``attn_decode`` entry (csrc/kernels/attention/decode.cu:4-67): one query
    token per sequence against ``k`` / ``v`` tensors, ``[batch, heads, len, 128]`` (layout 0) or
    ``[batch, len, heads, 128]`` (layout 1); the result has ``q``'s layout. ``causal_offset >= 0``
    limits the keys to ``0 .. causal_offset`` (layout_policies.cuh:138-141), ``mask`` (bool, True =
    attend) is ``[batch, kv_len]``, ``[batch, 1, kv_len]`` or ``[batch, 1 | heads, 1, kv_len]``. The split
    buffers are not needed. Layout 0 without a mask runs the dense-cache kernel in place; the
    other cases run the paged kernel over the token-major tensors (layout 0 is copied for it)."""
    b, q_len, kv_len, h, hkv, d = _dense_args(q, k, v, layout, "attn_decode")
    if q_len != 1:
        raise RuntimeError("Q seq_len must be 1")
    m4 = _dense_mask(mask, b, 1, kv_len, h)
    if d not in (32, 64, 128, 256) or h // hkv > 16:
        raise RuntimeError("attn_decode needs head_dim in (32, 64, 128, 256) and n_heads / n_kv_heads <= 16")
    attend = kv_len if causal_offset < 0 else min(kv_len, causal_offset + 1)
    with _on_device(q.device):
        if kv_len == 0 or b == 0:
            return torch.zeros_like(q)
        if layout == BHLD and m4 is None and k.is_contiguous() and v.is_contiguous() and d == 128 and h <= 64 \
                and h // hkv <= 8:
            pos = torch.full((1,), attend - 1, dtype=torch.int64, device=q.device)
            out = attn_decode(q.contiguous(), k, v, pos, scale=scale if scale > 0 else None)
            return out.reshape(b, h, 1, d)
        k_tm, v_tm = _token_major(k, layout), _token_major(v, layout)
        table, rows = _identity_paging(b, kv_len, q.device)
        indptr = (torch.arange(b + 1, dtype=torch.int32, device=q.device) * attend)
        q3, k_pool, v_pool = q.reshape(b, h, d), k_tm.view(b * kv_len, hkv, d), v_tm.view(b * kv_len, hkv, d)
        if m4 is not None and m4.size(1) != 1:
            # one mask row per head: only the general kernel addresses a mask by head
            mh = m4[:, :, 0]
            mh = mh if mh.stride(-1) == 1 else mh.contiguous()
            out = torch.empty((b, h, d), device=q.device, dtype=torch.bfloat16)
            nsplit = max(1, min(64, 2048 // max(1, b * hkv), kv_len // 64))
            _paged_rows(_require(), q3.contiguous(), k_pool, v_pool, table, rows, indptr, None,
                        (mh.data_ptr(), mh.stride(0), mh.stride(1), 0, 1, mh.size(2)), out, b, nsplit, False,
                        scale if scale > 0 else d ** -0.5)
            return out.reshape(q.shape)
        out = attn_paged_decode(q3, k_pool, v_pool, table, rows, indptr,
                                mask=None if m4 is None else m4[:, 0, 0], scale=scale)
    return out.reshape(q.shape)  # one token: both layouts have the same memory order


def attn_prefill_qkv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor] = None,
                     causal_offset: int = -1, scale: float = 0.0, layout: int = BHLD) -> torch.Tensor:
    """The reference's ``attn_prefill`` entry (csrc/kernels/attention/prefill.cu): a block of
    query rows per sequence against ``k`` / ``v`` tensors in either layout; the result has
    ``q``'s layout. ``causal_offset >= 0``: row ``i`` sees keys ``0 .. i + causal_offset``
    (prefill_split_q_mma.cuh:121-124); ``mask`` (bool, True = attend) is ``[batch, kv_len]``,
    ``[batch, 1 | q_len, kv_len]`` or ``[batch, 1 | heads, 1 | q_len, kv_len]``. Layout 0 without
    a mask runs the dense-cache kernel in place; the other cases run the ragged paged kernel
    over the token-major tensors (layout 0 is copied for it); an offset other than
    ``kv_len - q_len`` is expressed through the mask."""
    b, q_len, kv_len, h, hkv, d = _dense_args(q, k, v, layout, "attn_prefill")
    m4 = _dense_mask(mask, b, q_len, kv_len, h)
    if d not in (32, 64, 128, 256) or h // hkv > 16:
        raise RuntimeError("attn_prefill needs head_dim in (32, 64, 128, 256) and n_heads / n_kv_heads <= 16")
    with _on_device(q.device):
        if kv_len == 0 or b == 0 or q_len == 0:
            return torch.zeros_like(q)
        rows_i = torch.arange(q_len, dtype=torch.int64, device=q.device)
        if layout == BHLD and m4 is None and k.is_contiguous() and v.is_contiguous() and attn_prefill_supported(h, hkv, d):
            pos = torch.full_like(rows_i, kv_len - 1) if causal_offset < 0 else (rows_i + causal_offset).clamp_max(kv_len - 1)
            out = attn_prefill(q.contiguous(), k, v, pos, scale=scale if scale > 0 else None)
            return out.view(b, q_len, h, d).transpose(1, 2)
        causal = causal_offset >= 0 and causal_offset == kv_len - q_len
        if causal_offset >= 0 and not causal:
            band = torch.arange(kv_len, device=q.device)[None, :] <= (rows_i + causal_offset)[:, None]
            band = band[None, None].expand(b, 1, q_len, kv_len)
            m4 = band if m4 is None else (m4 & band)
        q_tm = _token_major(q, layout)
        k_tm, v_tm = _token_major(k, layout), _token_major(v, layout)
        table, rows = _identity_paging(b, kv_len, q.device)
        key = ("sched", b, q_len, str(q.device))
        if key not in _index_cache:
            _index_cache[key] = paged_prefill_schedule([q_len] * b, q.device)
        qo, tb, ti = _index_cache[key]
        kvp = torch.arange(b + 1, dtype=torch.int32, device=q.device) * kv_len
        out = attn_paged_prefill(q_tm.view(b * q_len, h, d), k_tm.view(b * kv_len, hkv, d),
                                 v_tm.view(b * kv_len, hkv, d), table, rows, kvp, qo, tb, ti, mask=m4,
                                 causal_offset=0 if causal else -1, scale=scale)
    out = out.view(b, q_len, h, d)
    return out if layout == BLHD else out.transpose(1, 2)

