"""Stateless adapters over the C-ABI kernels. The attention and rotary entry points that the
reference exports from ``astrai/extension/ops/__init__.py`` are re-exported here under the same
names; the quantized-GEMM custom ops live in the ``fp8``, ``fp8_block`` and ``int8`` modules
beside this file."""

from astrai_amd.extension.ops import attention as _attention
from astrai_amd.extension.ops import rotary as _rotary

_EXPORTS = {
    _attention: ("TensorLayout", "attn_decode", "attn_prefill", "attn_paged_decode", "attn_paged_prefill"),
    _rotary: ("rotary_emb",),
}
for _module, _names in _EXPORTS.items():
    for _name in _names:
        globals()[_name] = getattr(_module, _name)

__all__ = sorted(n for names in _EXPORTS.values() for n in names)
