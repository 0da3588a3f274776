"""int8 W8A8 linear policy: weights quantized once per output channel and
cached, activations quantized per token on every call, every ``F.linear`` on
bf16 GPU tensors routed through the int8 kernels while enabled.

The reference has no int8 policy; this follows the shape of its fp8 one
(astrai/extension/fp8.py:193-262,338-372): a process-global state object, an
autocast-style context manager, an enable switch, and a guard that falls
through to the stock kernel for anything it does not take. The per-weight cache
is keyed like the reference's per-weight metas, ``(data_ptr, shape, dtype)``
(fp8.py:200-208); an entry also holds a weak reference to the tensor object it
was made for and that tensor's version, so an in-place update re-quantizes and
a new tensor that lands on a freed weight's address never gets the old codes.
"""

import weakref
from contextlib import contextmanager
from typing import Dict, Optional, Tuple

import torch

from astrai_amd.extension import dispatch
from astrai_amd.extension.ops.int8 import (
    linear_forward_int8,
    quantize_int8_per_channel,
)


class Int8State:
    def __init__(self):
        self.enabled = False
        # key -> (weakref to the weight, its version, wq, sw)
        self._weights: Dict[Tuple, Tuple[weakref.ref, int, torch.Tensor, torch.Tensor]] = {}

    @staticmethod
    def _key(w: torch.Tensor) -> Tuple:
        return (w.data_ptr(), w.shape, w.dtype)

    def _store(self, w: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor) -> None:
        dead = [k for k, e in self._weights.items() if e[0]() is None]
        for k in dead:
            del self._weights[k]
        self._weights[self._key(w)] = (weakref.ref(w), w._version, wq, sw)

    def lookup(self, w: torch.Tensor) -> Optional[Tuple[torch.Tensor, torch.Tensor]]:
        """The cached ``(wq, sw)`` of this very tensor object at its current
        version, or ``None``."""
        hit = self._weights.get(self._key(w))
        if hit is not None and hit[0]() is w and hit[1] == w._version:
            return hit[2], hit[3]
        return None

    def get_weight(self, w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """``(wq int8 [N,K], sw fp32 [N])`` for ``w``, quantizing on first use."""
        hit = self.lookup(w)
        if hit is not None:
            return hit
        wq, sw = quantize_int8_per_channel(w.detach())
        self._store(w, wq, sw)
        return wq, sw

    def put_weight(self, w: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor) -> None:
        """Install an already quantized form of ``w`` (e.g. from an int8 checkpoint)."""
        if wq.shape != w.shape or wq.dtype != torch.int8 or sw.numel() != w.size(0):
            raise ValueError("wq must be int8 of w's shape and sw one step per output channel")
        self._store(w, wq.contiguous(), sw.reshape(-1).float().contiguous())

    def reset(self) -> None:
        self.enabled = False
        self._weights.clear()


_state = Int8State()


def int8_state() -> Int8State:
    return _state


def int8_linear_enable(enabled: bool = True) -> None:
    _state.enabled = enabled


def int8_linear_enabled() -> bool:
    return _state.enabled


@contextmanager
def int8_autocast(enabled: bool = True):
    prev = _state.enabled
    _state.enabled = enabled
    try:
        yield
    finally:
        _state.enabled = prev


def prepare_int8_weights(module: torch.nn.Module) -> int:
    """Quantize every 2-D bf16 GPU ``weight`` that an ``F.linear`` call inside
    ``module`` would hit, ahead of the first forward (so that a captured graph
    never contains the one-off weight pass). Returns the number of weights."""
    n = 0
    for mod in module.modules():
        w = getattr(mod, "weight", None)
        if (
            isinstance(w, torch.Tensor)
            and w.dim() == 2
            and w.is_cuda
            and w.dtype == torch.bfloat16
            and not isinstance(mod, torch.nn.Embedding)
            and type(mod).__name__ != "Embedding"
        ):
            _state.get_weight(w)
            n += 1
    return n


def int8_linear_forward(x: torch.Tensor, w: torch.Tensor, bias=None) -> torch.Tensor:
    wq, sw = _state.get_weight(w)
    b = bias if (bias is not None and bias.numel()) else None
    return linear_forward_int8(x, wq, sw, b)


def _int8_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    return x.dim() >= 1 and w.dim() == 2 and x.size(-1) == w.size(1) and x.numel() > 0


def _int8_handler(x, w, bias):
    if (
        _state.enabled
        and x.dtype == torch.bfloat16
        and w.dtype == torch.bfloat16
        and (bias is None or bias.dtype == torch.bfloat16)
        and _int8_supported(x, w)
    ):
        return int8_linear_forward(x, w, bias)
    return None


dispatch.register_handler(_int8_handler)
