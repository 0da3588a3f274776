"""int8 W8A8 (per-token x per-channel) op adapter. The reference has no int8
path; these ops follow the shape of its fp8 adapter (astrai/extension/ops/fp8.py):
stateless primitives over the registry module, custom ops with fake kernels,
scales as quantization steps.

- ``quantize_int8_per_token(x) -> (xq [M,K] int8, sx [M,1] fp32)``
- ``mm_int8(xq, wq, sx, sw, bias=None) -> bf16 [M,N]``  (``xq @ wq^T * sx[m] * sw[n] + bias``)
- ``mm_int8_acc(xq, wq) -> int32 [M,N]``  (raw accumulator, the bit-exact parity surface)
- ``linear_forward_int8(x, wq, sw, bias=None) -> bf16 [..., N]``
- ``rmsnorm_quantize_int8(x, weight, eps, res=None) -> (xq, sx, x + res | None)``: the
  residual add, ``F.rms_norm`` and the per-token quantizer in one kernel
- ``silu_mul_quantize_int8(gate, up) -> (hq, sh)``: ``up * silu(gate)`` and the
  per-token quantizer in one kernel
- ``mm_int8_swiglu(xq, wgu, sx, sgu) -> (hq, sh)``: the gate and up projections (one weight
  in ``swiglu_block_rows`` order), the SwiGLU product and the per-token quantizer; large
  shapes form ``h`` in the GEMM's epilogue, gate|up never reaches memory
"""

from typing import Optional

import torch
from torch.library import custom_op

from astrai_amd.extension.loader import get_module, is_available

_MOD: Optional[object] = None


def _mod() -> object:
    global _MOD
    if _MOD is None:
        if not is_available("int8_mm"):
            raise RuntimeError(
                "HIP kernel 'int8_mm' is not available. Build with `make -C astrai_amd/csrc`."
            )
        _MOD = get_module("int8_mm")
    return _MOD


def _no_cpu(op: str):
    raise RuntimeError(
        f"{op}: this backend has no CPU implementation; pass tensors on the MI355X device"
    )


@custom_op("custom::int8_quantize_per_token", mutates_args=())
def int8_quantize_per_token(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """bf16 ``[..., K]`` -> ``(xq int8 [R,K], s fp32 [R,1])``, symmetric, one step per row."""
    _no_cpu("custom::int8_quantize_per_token")


@int8_quantize_per_token.register_fake
def _int8_quantize_fake(x):
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    return (
        torch.empty((rows, k), device=x.device, dtype=torch.int8),
        torch.empty((rows, 1), device=x.device, dtype=torch.float32),
    )


@int8_quantize_per_token.register_kernel("cuda")
def _int8_quantize_cuda(x):
    if x.dtype != torch.bfloat16:
        raise TypeError(f"int8 quantize requires bf16 input, got {x.dtype}")
    return _mod().quantize_int8_rows(x)


@custom_op("custom::int8_gemm", mutates_args=())
def int8_gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    sa: torch.Tensor,
    sb: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """int8 GEMM ``a @ b^T`` (exact int32) scaled by ``sa[m] * sb[n]``, optional bias, bf16 out."""
    _no_cpu("custom::int8_gemm")


@int8_gemm.register_fake
def _int8_gemm_fake(a, b, sa, sb, bias=None):
    return torch.empty((a.size(0), b.size(0)), device=a.device, dtype=torch.bfloat16)


@int8_gemm.register_kernel("cuda")
def _int8_gemm_cuda(a, b, sa, sb, bias=None):
    if a.dtype != torch.int8 or b.dtype != torch.int8:
        raise TypeError(f"int8 GEMM requires int8 inputs, got {a.dtype}/{b.dtype}")
    return _mod().mm_int8(a, b, sa, sb, bias, 0)


def quantize_int8_per_token(x: torch.Tensor):
    return int8_quantize_per_token(x)


def quantize_int8_per_channel(w: torch.Tensor):
    """Weights ``[N,K]`` -> ``(wq int8 [N,K], sw fp32 [N])``: the per-row quantizer on W."""
    if w.dim() != 2:
        raise ValueError("weight must be 2D [N, K]")
    wq, s = int8_quantize_per_token(w)
    return wq, s.reshape(-1)


def mm_int8(xq, wq, sx, sw, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    return int8_gemm(xq, wq, sx, sw, bias)


@custom_op("custom::int8_gemm_resid", mutates_args=())
def int8_gemm_resid(xq: torch.Tensor, wq: torch.Tensor, sx: torch.Tensor, sw: torch.Tensor,
                    resid: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``int8_gemm(xq, wq, sx, sw, bias) + resid`` in bf16 arithmetic: a projection whose
    output joins the residual stream (astrai/model/components/decoder_block.py:67,70)."""
    _no_cpu("custom::int8_gemm_resid")


@int8_gemm_resid.register_fake
def _int8_gemm_resid_fake(xq, wq, sx, sw, resid, bias=None):
    return torch.empty((xq.shape[0], wq.shape[0]), device=xq.device, dtype=torch.bfloat16)


@int8_gemm_resid.register_kernel("cuda")
def _int8_gemm_resid_cuda(xq, wq, sx, sw, resid, bias=None):
    return _mod().mm_int8_resid(xq, wq, sx, sw, resid, bias)


def mm_int8_resid(xq, wq, sx, sw, resid, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    return int8_gemm_resid(xq, wq, sx, sw, resid, bias)


def mm_int8_acc(xq: torch.Tensor, wq: torch.Tensor, kernel: str = "auto") -> torch.Tensor:
    """Raw int32 accumulator ``xq @ wq^T`` from the named kernel (auto / gemv / tiled)."""
    if xq.dtype != torch.int8 or wq.dtype != torch.int8:
        raise TypeError(f"int8 GEMM requires int8 inputs, got {xq.dtype}/{wq.dtype}")
    return _mod().mm_int8(xq, wq, None, None, None, 2, kernel)


def linear_forward_int8(x, wq, sw, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """W8A8 linear forward: per-token quantize ``x`` (bf16), int8 GEMM against the
    pre-quantized weight, dequant epilogue. ``x`` is ``[..., K]``; returns ``[..., N]``."""
    if x.dtype != torch.bfloat16:
        raise TypeError(f"int8 forward requires bf16 activations, got {x.dtype}")
    xq, sx = int8_quantize_per_token(x)
    out = int8_gemm(xq, wq, sx, sw, bias)
    return out.reshape(*x.shape[:-1], wq.size(0))


@custom_op("custom::int8_add_rmsnorm_quantize", mutates_args=())
def int8_add_rmsnorm_quantize(
    x: torch.Tensor, weight: torch.Tensor, eps: float, res: Optional[torch.Tensor] = None
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``t = x + res`` (``x`` itself without ``res``), ``y = rms_norm(t) * weight``,
    per-token int8 of ``y``. Returns ``(xq int8 [R,K], s fp32 [R,1], t)``."""
    _no_cpu("custom::int8_add_rmsnorm_quantize")


@int8_add_rmsnorm_quantize.register_fake
def _int8_add_rmsnorm_quantize_fake(x, weight, eps, res=None):
    k = x.shape[-1]
    rows = x.numel() // k if k else 0
    return (
        torch.empty((rows, k), device=x.device, dtype=torch.int8),
        torch.empty((rows, 1), device=x.device, dtype=torch.float32),
        torch.empty_like(x),
    )


@int8_add_rmsnorm_quantize.register_kernel("cuda")
def _int8_add_rmsnorm_quantize_cuda(x, weight, eps, res=None):
    if x.dtype != torch.bfloat16:
        raise TypeError(f"int8 rmsnorm-quantize requires bf16 input, got {x.dtype}")
    xq, s, t, _ = _mod().add_rmsnorm_quantize_int8(x, weight, eps, res, False)
    # a custom op may not return an input: without a residual the sum is a copy of x
    return xq, s, (t if t is not None else x.clone())


@custom_op("custom::int8_silu_mul_quantize", mutates_args=())
def int8_silu_mul_quantize(gate: torch.Tensor, up: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``h = up * silu(gate)`` in bf16 arithmetic, per-token int8 of ``h``:
    ``(hq int8 [R,W], s fp32 [R,1])``."""
    _no_cpu("custom::int8_silu_mul_quantize")


@int8_silu_mul_quantize.register_fake
def _int8_silu_mul_quantize_fake(gate, up):
    w = gate.shape[-1]
    rows = gate.numel() // w if w else 0
    return (
        torch.empty((rows, w), device=gate.device, dtype=torch.int8),
        torch.empty((rows, 1), device=gate.device, dtype=torch.float32),
    )


@int8_silu_mul_quantize.register_kernel("cuda")
def _int8_silu_mul_quantize_cuda(gate, up):
    if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16:
        raise TypeError(f"int8 silu-mul-quantize requires bf16 inputs, got {gate.dtype}/{up.dtype}")
    hq, s, _ = _mod().silu_mul_quantize_int8(gate, up, False)
    return hq, s


def rmsnorm_quantize_int8(x, weight, eps: float, res: Optional[torch.Tensor] = None):
    """Fused (residual add +) RMSNorm + per-token int8. Returns ``(xq, sx, t)`` with
    ``t = x + res`` when ``res`` is given, else ``None`` (no copy is made)."""
    if x.dtype != torch.bfloat16:
        raise TypeError(f"int8 rmsnorm-quantize requires bf16 input, got {x.dtype}")
    xq, s, t, _ = _mod().add_rmsnorm_quantize_int8(x, weight, eps, res, False)
    return xq, s, t


def silu_mul_quantize_int8(gate, up):
    return int8_silu_mul_quantize(gate, up)


@custom_op("custom::int8_mm_swiglu", mutates_args=())
def int8_mm_swiglu(xq: torch.Tensor, wgu: torch.Tensor, sx: torch.Tensor,
                   sgu: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """``h = up(x) * silu(gate(x))`` (astrai/model/components/mlp.py:40-43) from int8 ``xq
    [M,K]`` and the blocked gate|up weight ``wgu [2W,K]``, per-token int8 of ``h``:
    ``(hq int8 [M,W], s fp32 [M,1])``."""
    _no_cpu("custom::int8_mm_swiglu")


@int8_mm_swiglu.register_fake
def _int8_mm_swiglu_fake(xq, wgu, sx, sgu):
    m, w = xq.shape[0], wgu.shape[0] // 2
    return (
        torch.empty((m, w), device=xq.device, dtype=torch.int8),
        torch.empty((m, 1), device=xq.device, dtype=torch.float32),
    )


@int8_mm_swiglu.register_kernel("cuda")
def _int8_mm_swiglu_cuda(xq, wgu, sx, sgu):
    hq, s, _ = _mod().mm_int8_swiglu(xq, wgu, sx, sgu, False)
    return hq, s


def mm_int8_swiglu(xq, wgu, sx, sgu):
    return int8_mm_swiglu(xq, wgu, sx, sgu)


def swiglu_block_rows(gate, up):
    """Gate and up rows (weights or their scales) in the order ``mm_int8_swiglu`` takes."""
    return _mod().swiglu_block_rows(gate, up)
