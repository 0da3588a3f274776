"""Kernel registry: the same three public names as the reference's
``astrai/extension/loader.py`` (``KERNEL_NAMES``, ``is_available``,
``get_module``, loader.py:23-54).

The reference globs ``lib/*.so`` and imports each file as a pybind module. The
MI355X backend is one plain C-ABI library (no ``PyInit_*``), so the registry
binds it with ctypes and exposes, per kernel name, an adapter object carrying
the callables the pybind module of that name carries. A kernel whose library is
absent is reported unavailable (``False`` / ``None``), never by an exception at
import, exactly as the reference does (loader.py:36-44).
"""

from __future__ import annotations

import logging
from types import SimpleNamespace

from astrai_amd.extension import _cabi

logger = logging.getLogger(__name__)


def _fp8_mm_module() -> SimpleNamespace:
    # the five callables of csrc/kernels/fp8/mm.cu:350-369
    return SimpleNamespace(
        fp8_mm=_cabi.fp8_mm,
        quantize_bf16=_cabi.quantize_bf16,
        mm_fp8=_cabi.mm_fp8,
        linear_forward_fp8=_cabi.linear_forward_fp8,
        linear_backward_fp8=_cabi.linear_backward_fp8,
        mm_fp8_acc=_cabi.mm_fp8_acc,
        quantize_transpose_bf16=_cabi.quantize_transpose_bf16,
        amax_bf16=_cabi.amax_bf16,
        amax_ring_push=_cabi.amax_ring_push,
        new_amax_partials=_cabi.new_amax_partials,
        quantize_bf16_partials=_cabi.quantize_bf16_partials,
        amax_bf16_partials=_cabi.amax_bf16_partials,
        amax_ring_push_partials=_cabi.amax_ring_push_partials,
        add_rmsnorm_quantize_fp8=_cabi.add_rmsnorm_quantize_fp8,
        silu_mul_quantize_fp8=_cabi.silu_mul_quantize_fp8,
    )


def _int8_mm_module() -> SimpleNamespace:
    return SimpleNamespace(
        quantize_int8_rows=_cabi.quantize_int8_rows,
        mm_int8=_cabi.mm_int8,
        add_rmsnorm_quantize_int8=_cabi.add_rmsnorm_quantize_int8,
        silu_mul_quantize_int8=_cabi.silu_mul_quantize_int8,
        mm_int8_swiglu=_cabi.mm_int8_swiglu,
        mm_int8_resid=_cabi.mm_int8_resid,
        swiglu_block_rows=_cabi.swiglu_block_rows,
    )


def _fp8_block_mm_module() -> SimpleNamespace:
    return SimpleNamespace(
        quantize_fp8_block128_act=_cabi.quantize_fp8_block128_act,
        quantize_fp8_block128_weight=_cabi.quantize_fp8_block128_weight,
        mm_fp8_block128=_cabi.mm_fp8_block128,
    )


def _attn_paged_decode_module() -> SimpleNamespace:
    # the callable of csrc/kernels/attention/paged_decode.cu:69-86, same argument list
    return SimpleNamespace(attn_paged_decode=_cabi.attn_paged_decode)


def _attn_paged_prefill_module() -> SimpleNamespace:
    # the callable of csrc/kernels/attention/paged_prefill.cu:36-52, same argument list
    return SimpleNamespace(attn_paged_prefill=_cabi.attn_paged_prefill)


def _attn_decode_module() -> SimpleNamespace:
    # the callable of csrc/kernels/attention/decode.cu:4-67 (q, k, v tensors in either layout)
    return SimpleNamespace(attn_decode=_cabi.attn_decode_qkv)


def _attn_prefill_module() -> SimpleNamespace:
    # the callable of csrc/kernels/attention/prefill.cu, same argument list
    return SimpleNamespace(attn_prefill=_cabi.attn_prefill_qkv)


def _rotary_emb_module() -> SimpleNamespace:
    # the callable of csrc/kernels/rotary/rotary_emb.cu:47-93
    return SimpleNamespace(rotary_emb=_cabi.rotary_emb)


_FACTORIES = {
    "attn_decode": _attn_decode_module,
    "attn_prefill": _attn_prefill_module,
    "rotary_emb": _rotary_emb_module,
    "attn_paged_decode": _attn_paged_decode_module,
    "attn_paged_prefill": _attn_paged_prefill_module,
    "fp8_mm": _fp8_mm_module,
    "int8_mm": _int8_mm_module,
    "fp8_block_mm": _fp8_block_mm_module,
}

KERNEL_NAMES = sorted(_FACTORIES)

_available: dict[str, bool] = {}
_modules: dict[str, object] = {}

_loaded = _cabi.load() is not None
if not _loaded:
    logger.debug("libastrai_w8a8.so unavailable: %s", _cabi.load_error())
for _name in KERNEL_NAMES:
    _available[_name] = _loaded
    _modules[_name] = _FACTORIES[_name]() if _loaded else None


def is_available(name: str) -> bool:
    """Return ``True`` if the compiled kernel ``name`` was loaded."""
    return _available.get(name, False)


def get_module(name: str) -> object:
    """Return the loaded kernel module for ``name``, or ``None`` if unavailable."""
    return _modules.get(name)
