"""e4m3fn GEMM with 128-block scales (1x128 activation groups, 128x128 weight
blocks). Not in the reference; same adapter shape as astrai/extension/ops/fp8.py.

- ``quantize_act_block128(x) -> (x8 [M,K], sa [M,K/128])``
- ``quantize_weight_block128(w) -> (w8 [N,K], sb [ceil(N/128),K/128])``
- ``mm_fp8_blockscaled(a8, b8, sa, sb, bias=None) -> bf16 [M,N]``
"""

from typing import Optional

import torch
from torch.library import custom_op

from astrai_amd.extension.loader import get_module, is_available

_MOD: Optional[object] = None


def _mod() -> object:
    global _MOD
    if _MOD is None:
        if not is_available("fp8_block_mm"):
            raise RuntimeError(
                "HIP kernel 'fp8_block_mm' is not available. Build with `make -C astrai_amd/csrc`."
            )
        _MOD = get_module("fp8_block_mm")
    return _MOD


def _no_cpu(op: str):
    raise RuntimeError(
        f"{op}: this backend has no CPU implementation; pass tensors on the MI355X device"
    )


@custom_op("custom::fp8_gemm_blockscaled", mutates_args=())
def fp8_gemm_blockscaled(
    a: torch.Tensor,
    b: torch.Tensor,
    sa: torch.Tensor,
    sb: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``sum_kb (a8[:,kb] @ b8[:,kb]^T) * sa[m,kb] * sb[n/128,kb]`` in fp32, bf16 out."""
    _no_cpu("custom::fp8_gemm_blockscaled")


@fp8_gemm_blockscaled.register_fake
def _fake(a, b, sa, sb, bias=None):
    return torch.empty((a.size(0), b.size(0)), device=a.device, dtype=torch.bfloat16)


@fp8_gemm_blockscaled.register_kernel("cuda")
def _cuda(a, b, sa, sb, bias=None):
    if a.dtype != torch.float8_e4m3fn or b.dtype != torch.float8_e4m3fn:
        raise TypeError(f"block-scaled GEMM requires e4m3fn inputs, got {a.dtype}/{b.dtype}")
    return _mod().mm_fp8_block128(a, b, sa, sb, bias)


def quantize_act_block128(x: torch.Tensor):
    if x.dtype != torch.bfloat16:
        raise TypeError(f"block quantize requires bf16 input, got {x.dtype}")
    return _mod().quantize_fp8_block128_act(x)


def quantize_weight_block128(w: torch.Tensor):
    if w.dtype != torch.bfloat16:
        raise TypeError(f"block quantize requires bf16 input, got {w.dtype}")
    return _mod().quantize_fp8_block128_weight(w)


def mm_fp8_blockscaled(a8, b8, sa, sb, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    return fp8_gemm_blockscaled(a8, b8, sa, sb, bias)
