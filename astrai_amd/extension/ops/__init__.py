"""Stateless adapters over the C-ABI kernels: the attention and rotary entry points the
reference exports from ``astrai/extension/ops/__init__.py``; the quantized-GEMM custom ops
live in the ``fp8``, ``fp8_block`` and ``int8`` modules beside this file."""

from astrai_amd.extension.ops.attention import (
    TensorLayout,
    attn_decode,
    attn_paged_decode,
    attn_paged_prefill,
    attn_prefill,
)
from astrai_amd.extension.ops.rotary import rotary_emb

__all__ = [
    "TensorLayout",
    "attn_decode",
    "attn_paged_decode",
    "attn_paged_prefill",
    "attn_prefill",
    "rotary_emb",
]
