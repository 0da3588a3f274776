"""``aten::linear`` hook shared by the fp8 and int8 policies.

The reference installs a CUDA-key implementation of ``aten::linear`` when
``astrai.extension.fp8`` is imported (astrai/extension/fp8.py:404-406); ROCm
tensors carry the same dispatch key. Policies register a *handler*
``(x, w, bias) -> Tensor | None``; the first one that returns a tensor wins, and
when none does the call is re-dispatched to the stock composite kernel exactly
as the reference's guard does (fp8.py:367-372).
"""

from typing import Callable, List, Optional

import torch
from torch.library import Library

Handler = Callable[[torch.Tensor, torch.Tensor, Optional[torch.Tensor]], Optional[torch.Tensor]]

_handlers: List[Handler] = []
_backward_handlers: List[Callable] = []
_lib: Optional[Library] = None


def _stock_linear(x, w, bias):
    return torch.ops.aten.linear.default.redispatch(
        torch._C.DispatchKeySet(torch._C.DispatchKey.CompositeImplicitAutograd), x, w, bias
    )


def _linear_cuda_impl(x: torch.Tensor, w: torch.Tensor, bias=None):
    for h in _handlers:
        out = h(x, w, bias)
        if out is not None:
            return out
    return _stock_linear(x, w, bias)


def _linear_backward_cuda_impl(input_tensor, grad_output, weight, output_mask):
    """Overriding ``linear`` on the CUDA key makes autograd call
    ``aten::linear_backward``, which has no stock CUDA kernel; policies may take
    it (fp8 backward), otherwise this is the plain matmul form the reference
    falls back to (fp8.py:382-401)."""
    for h in _backward_handlers:
        out = h(input_tensor, grad_output, weight, output_mask)
        if out is not None:
            return out
    dt = weight.dtype
    grad = grad_output.to(dt)
    g2 = grad.reshape(-1, weight.size(0))
    x2 = input_tensor.reshape(-1, input_tensor.size(-1)).to(dt)

    def none():
        return torch.empty(0, device=input_tensor.device, dtype=input_tensor.dtype)

    gi = torch.mm(g2, weight) if output_mask[0] else none()
    gw = torch.mm(g2.t(), x2) if output_mask[1] else none()
    gb = g2.sum(dim=0) if output_mask[2] else none()
    return (gi.reshape_as(input_tensor) if output_mask[0] else gi), gw, gb


def install() -> None:
    """Install the override once per process."""
    global _lib
    if _lib is None:
        _lib = Library("aten", "IMPL", "CUDA")
        _lib.impl("linear", _linear_cuda_impl)
        _lib.impl("linear_backward", _linear_backward_cuda_impl)


def register_handler(h: Handler, backward: Optional[Callable] = None) -> None:
    if h not in _handlers:
        _handlers.append(h)
    if backward is not None and backward not in _backward_handlers:
        _backward_handlers.append(backward)
    install()
