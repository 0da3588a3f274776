"""FP8 scaling policy and ``aten::linear`` integration -- the counterpart of the
reference's ``astrai/extension/fp8.py`` with the same public names:

``FP8_MAX``, ``FP8Format``, ``FP8Recipe``, ``DelayedScaling``, ``DynamicScaling``,
``FP8TensorMeta``, ``FP8State``, ``fp8_state``, ``fp8_autocast``,
``fp8_linear_forward``, ``fp8_linear_backward``, ``fp8_linear_enable``,
``fp8_linear_enabled``.

Usage (unchanged from the reference)::

    from astrai_amd.extension.fp8 import fp8_autocast
    with fp8_autocast(enabled=True, fp8_format="hybrid"):
        logits = model(input_ids)      # every F.linear on bf16 GPU tensors -> fp8 kernels

Scales are quantization steps derived from amax: ``scale = amax / FP8_MAX[fmt] /
2**margin``, floored at 1e-12 (fp8.py:87-89,103-105). All policy arithmetic
stays on the device as tiny tensor ops; nothing here reads a value back to the
host, so the path stays stream-ordered and graph-capturable.
"""

import weakref
from contextlib import contextmanager
from dataclasses import dataclass
from enum import Enum
from typing import Dict, Optional, Tuple

import torch

from astrai_amd.extension import dispatch
from astrai_amd.extension.ops.fp8 import (
    amax_bf16,
    amax_bf16_partials,
    amax_ring_push,
    amax_ring_push_partials,
    linear_backward_fp8,
    linear_forward_fp8,
    mm_fp8,
    mm_fp8_bias,
    new_amax_partials,
    quantize_bf16,
    quantize_bf16_partials,
)

FP8_MAX = {"e4m3": 448.0, "e5m2": 57344.0}
E4M3_MAX = FP8_MAX["e4m3"]
_FLOOR = 1e-12


class FP8Format(str, Enum):
    """Format per direction; HYBRID = E4M3 forward, E5M2 backward (fp8.py:47-58)."""

    E4M3 = "e4m3"
    E5M2 = "e5m2"
    HYBRID = "hybrid"

    def fwd(self) -> str:
        return "e4m3" if self is FP8Format.HYBRID else self.value

    def bwd(self) -> str:
        return "e5m2" if self is FP8Format.HYBRID else self.value


def _step(peak: torch.Tensor, fmt: str, margin: int) -> torch.Tensor:
    return ((peak / FP8_MAX[fmt]) / (2**margin)).clamp_min(_FLOOR)


class FP8Recipe:
    """Maps an amax window to a quantization step (fp8.py:61-76)."""

    history_len: int = 16
    margin: int = 0

    def scale_from_history(self, amax: torch.Tensor, fmt: str) -> torch.Tensor:
        raise NotImplementedError


@dataclass
class DelayedScaling(FP8Recipe):
    """Max over the last ``history_len`` recorded amax values (fp8.py:79-92)."""

    history_len: int = 16
    margin: int = 0

    def scale_from_history(self, amax: torch.Tensor, fmt: str) -> torch.Tensor:
        return _step(amax.max(), fmt, self.margin)


@dataclass
class DynamicScaling(FP8Recipe):
    """Scale from the amax of the tensor being quantized right now (fp8.py:95-108)."""

    history_len: int = 1
    margin: int = 0

    def scale_from_history(self, amax: torch.Tensor, fmt: str) -> torch.Tensor:
        return _step(amax.max(), fmt, self.margin)


class _AmaxRing:
    """One operand's amax history, write cursor, derived step and seeded flag."""

    __slots__ = ("hist", "idx", "scale", "seeded", "_partials")

    def __init__(self, device: torch.device, n: int):
        self.hist = torch.ones(n, device=device, dtype=torch.float32)
        self.scale = torch.ones(1, device=device, dtype=torch.float32)
        self.idx = 0
        self.seeded = False
        self._partials = None

    def takes_partials(self, recipe: FP8Recipe) -> bool:
        """The fast bookkeeping applies: device ring, a stock recipe (both take the window's
        maximum)."""
        return self.hist.is_cuda and type(recipe) in (DelayedScaling, DynamicScaling)

    @property
    def partials(self) -> torch.Tensor:
        """Scratch through which a quantizer hands this ring the amax it saw, as one maximum
        per workgroup (no slot to clear, no atomics); made on first use."""
        if self._partials is None:
            self._partials = new_amax_partials(self.hist.device)
        return self._partials

    def push_partials(self, recipe: FP8Recipe, fmt: str) -> None:
        """:meth:`push` of the amax a quantizer has just left in :attr:`partials`."""
        amax_ring_push_partials(self.hist, self.idx, self.partials, self.scale, FP8_MAX[fmt],
                                float(2 ** recipe.margin))
        self.idx = (self.idx + 1) % self.hist.numel()

    def push(self, amax: torch.Tensor, recipe: FP8Recipe, fmt: str) -> None:
        # record first, then refresh: the step used next reflects amax seen so far
        if self.hist.is_cuda and type(recipe) in (DelayedScaling, DynamicScaling) \
                and amax.is_cuda and amax.dtype == torch.float32 and amax.is_contiguous():
            # both stock recipes take the window's maximum: one launch does the lot
            amax_ring_push(self.hist, self.idx, amax, self.scale, FP8_MAX[fmt],
                           float(2 ** recipe.margin))
            self.idx = (self.idx + 1) % self.hist.numel()
            return
        self.hist[self.idx] = amax.reshape(())
        self.idx = (self.idx + 1) % self.hist.numel()
        self.scale.copy_(recipe.scale_from_history(self.hist, fmt))

    def seed(self, t: torch.Tensor, recipe: FP8Recipe, fmt: str) -> None:
        self.hist.fill_(t.abs().amax().to(torch.float32).clamp_min(_FLOOR))
        self.scale.copy_(recipe.scale_from_history(self.hist, fmt))
        self.seeded = True


def _ring_property(ring: str, field: str):
    def fget(self):
        return getattr(getattr(self, ring), field)

    def fset(self, value):
        setattr(getattr(self, ring), field, value)

    return property(fget, fset)


class FP8TensorMeta:
    """Per-weight scaling state: rings for weight / activation / gradient
    (fp8.py:111-190). Attribute names match the reference
    (``w_hist, w_idx, w_scale, w_init`` and the x_/g_ twins)."""

    def __init__(self, device: torch.device, recipe: FP8Recipe):
        self.recipe = recipe
        n = recipe.history_len
        self._w = _AmaxRing(device, n)
        self._x = _AmaxRing(device, n)
        self._g = _AmaxRing(device, n)
        # host-side bookkeeping of FP8State.cache_weights
        self.w_ref = None     # weakref to the tensor object whose pushes are being counted
        self.w_version = -1   # weight._version at the last push into the weight ring
        self.w_repeats = 0    # consecutive pushes made from that same version
        self.w_cached = None  # (weakref to the weight, version, w8, amax_w): codes made with the settled step

    w_hist, w_idx = _ring_property("_w", "hist"), _ring_property("_w", "idx")
    w_scale, w_init = _ring_property("_w", "scale"), _ring_property("_w", "seeded")
    x_hist, x_idx = _ring_property("_x", "hist"), _ring_property("_x", "idx")
    x_scale, x_init = _ring_property("_x", "scale"), _ring_property("_x", "seeded")
    g_hist, g_idx = _ring_property("_g", "hist"), _ring_property("_g", "idx")
    g_scale, g_init = _ring_property("_g", "scale"), _ring_property("_g", "seeded")

    def update_w(self, amax: torch.Tensor, fmt: str) -> None:
        self._w.push(amax, self.recipe, fmt)

    def update_x(self, amax: torch.Tensor, fmt: str) -> None:
        self._x.push(amax, self.recipe, fmt)

    def update_g(self, amax: torch.Tensor, fmt: str) -> None:
        self._g.push(amax, self.recipe, fmt)

    def init_w(self, w: torch.Tensor, fmt: str) -> None:
        self._w.seed(w, self.recipe, fmt)
        self.w_ref = weakref.ref(w)
        self.w_version, self.w_repeats = w._version, self.recipe.history_len

    def _same_weight(self, w: torch.Tensor) -> bool:
        # same tensor object (an address can be reused by another tensor), same contents
        return self.w_ref is not None and self.w_ref() is w and self.w_version == w._version

    def w_settled(self, w: torch.Tensor) -> bool:
        """True when every slot of the weight ring holds the amax of ``w`` as it is
        now, so that one more push would change neither the ring nor the step."""
        return self._same_weight(w) and self.w_repeats >= self.recipe.history_len

    def note_w_push(self, w: torch.Tensor) -> None:
        self.w_cached = None  # the step may have moved with this push
        if self._same_weight(w):
            self.w_repeats += 1
        else:
            self.w_ref, self.w_version, self.w_repeats = weakref.ref(w), w._version, 1

    def init_x(self, x: torch.Tensor, fmt: str) -> None:
        self._x.seed(x, self.recipe, fmt)

    def init_g(self, g: torch.Tensor, fmt: str) -> None:
        self._g.seed(g, self.recipe, fmt)


class FP8State:
    """Process-global switch, recipe, format and the per-weight metas (fp8.py:193-213).
    Global rather than thread-local because autograd's backward runs on engine threads."""

    def __init__(self):
        self.enabled = False
        self.recipe: FP8Recipe = DelayedScaling()
        self.fp8_format: FP8Format = FP8Format.HYBRID
        self._metas: Dict[Tuple, FP8TensorMeta] = {}
        self._last_device: Optional[torch.device] = None
        # Weight-code cache (fp8_cache_weights): keep each weight's fp8 codes between calls
        # for as long as the tensor's version counter stands still, instead of measuring
        # and quantizing the weight again in every forward (fp8.py:291-299 does). Outputs
        # and ring state are unchanged. None (the default) decides per call: on where no
        # optimizer can be rewriting the weight between forwards -- autograd is off, or the
        # weight takes no gradient --, off in a training step, where a write that bypasses
        # the version counter (``w.data`` tricks of some optimizers) would go unseen.
        self.cache_weights: Optional[bool] = None
        self._dyn_w: Dict[Tuple, Tuple] = {}
        self._scratch: Dict[Tuple, Tuple] = {}

    def get_weight_meta(self, w: torch.Tensor) -> FP8TensorMeta:
        key = (w.data_ptr(), w.shape, w.dtype)
        meta = self._metas.get(key)
        if meta is None:
            if self._last_device is None:
                self._last_device = w.device
            meta = self._metas[key] = FP8TensorMeta(w.device, self.recipe)
        return meta

    def peek_weight_meta(self, w: torch.Tensor) -> Optional[FP8TensorMeta]:
        """The scaling state of ``w`` if it has any; never creates one."""
        return self._metas.get((w.data_ptr(), w.shape, w.dtype))

    def dynamic_weight(self, w: torch.Tensor, fmt: str):
        """``(sw, w8)`` of dynamic scaling, reused while ``w`` is unmodified."""
        key = (w.data_ptr(), w.shape, fmt, self.recipe.margin)
        hit = self._dyn_w.get(key)
        # the entry must belong to this very tensor object: an address can be handed to a new
        # tensor whose version counter happens to match
        if hit is not None and hit[0]() is w and hit[1] == w._version:
            return hit[2], hit[3]
        sw = _dynamic_scale(w, self.recipe, fmt)
        w8, _ = quantize_bf16(w, sw, fmt)
        self._dyn_w[key] = (weakref.ref(w), w._version, sw, w8)
        return sw, w8

    def scratch(self, device: torch.device):
        """``(partials, slot)`` of dynamic scaling on ``device`` and the current stream: the
        per-workgroup maxima of the tensor being measured and a ring of one to push them
        through. Per stream, because a measurement and its push are ordered by the stream only."""
        key = (device, torch.cuda.current_stream(device).cuda_stream)
        hit = self._scratch.get(key)
        if hit is None:
            hit = self._scratch[key] = (new_amax_partials(device),
                                        torch.zeros(1, device=device, dtype=torch.float32))
        return hit

    def caches_weight(self, w: torch.Tensor) -> bool:
        if self.cache_weights is not None:
            return self.cache_weights
        return not (torch.is_grad_enabled() and w.requires_grad)

    def reset(self) -> None:
        self.enabled = False
        self.cache_weights = None
        self._metas.clear()
        self._dyn_w.clear()
        self._scratch.clear()
        self._last_device = None


_state = FP8State()


def fp8_state() -> FP8State:
    return _state


@contextmanager
def fp8_autocast(
    enabled: bool = True,
    update_interval: int = 16,
    recipe: Optional[FP8Recipe] = None,
    fp8_format: str = "hybrid",
    margin: int = 0,
):
    """Route ``aten::linear`` through the fp8 kernels inside the block; the
    previous (enabled, recipe, format) triple is restored on exit (fp8.py:226-262).
    ``update_interval`` / ``margin`` parametrise the default delayed recipe."""
    st = fp8_state()
    saved = (st.enabled, st.recipe, st.fp8_format)
    st.enabled = enabled
    st.recipe = recipe if recipe is not None else DelayedScaling(update_interval, margin)
    st.fp8_format = FP8Format(fp8_format)
    try:
        yield
    finally:
        st.enabled, st.recipe, st.fp8_format = saved


def _dynamic_scale(t: torch.Tensor, recipe: FP8Recipe, fmt: str) -> torch.Tensor:
    if t.is_cuda and t.dtype == torch.bfloat16:
        if type(recipe) in (DelayedScaling, DynamicScaling) and t.numel():
            # one read of t (no |t| temporary) leaves one maximum per workgroup; a window of
            # one then turns them into max((amax / FP8_MAX) / 2^margin, floor) in one launch
            # (flooring amax first, as the host formula does, cannot change that)
            st = fp8_state()
            partials, slot = st.scratch(t.device)
            scale = torch.empty(1, device=t.device, dtype=torch.float32)
            amax_bf16_partials(t, partials)
            amax_ring_push_partials(slot, 0, partials, scale, FP8_MAX[fmt], float(2 ** recipe.margin))
            return scale
        amax = amax_bf16(t).reshape(()).clamp_min(_FLOOR)
    else:
        amax = t.abs().amax().to(torch.float32).clamp_min(_FLOOR)
    return recipe.scale_from_history(amax, fmt)


def fp8_linear_forward(x: torch.Tensor, w: torch.Tensor, bias=None):
    """Scaled fp8 linear forward (fp8.py:275-305).

    Dynamic scaling: measure both operands, quantize, pre-quantized GEMM to bf16,
    then add the bias in bf16 (two roundings, as the reference does). Delayed
    scaling: quantize with the rings' current steps inside the fused forward,
    then push the returned amax values."""
    st = fp8_state()
    fmt = st.fp8_format.fwd()
    meta = st.get_weight_meta(w)
    if not meta.w_init:
        meta.init_w(w, fmt)
    if isinstance(st.recipe, DynamicScaling):
        x2 = x.reshape(-1, w.size(1))
        sx = _dynamic_scale(x2, st.recipe, fmt)
        x8, _ = quantize_bf16(x2, sx, fmt)
        if st.caches_weight(w):
            sw, w8 = st.dynamic_weight(w, fmt)
        else:
            sw = _dynamic_scale(w, st.recipe, fmt)
            w8, _ = quantize_bf16(w, sw, fmt)
        out = mm_fp8(x8, w8, sx, sw).reshape(*x.shape[:-1], w.size(0))
        if bias is not None and bias.numel():
            out = out + bias
        return out
    if not meta.x_init:
        meta.init_x(x, fmt)
    if st.caches_weight(w) and meta.w_settled(w):
        # The weight ring already holds this weight's amax in every slot: pushing it
        # again would leave ring and step as they are, so codes made with that step
        # stay valid until the weight is written to.
        hit = meta.w_cached
        if hit is None or hit[0]() is not w or hit[1] != w._version:
            w8, amax_w = quantize_bf16(w, meta.w_scale, "e4m3")
            meta.w_cached = (weakref.ref(w), w._version, w8, amax_w)
        x2 = x.reshape(-1, w.size(1))
        has_bias = bias is not None and bias.numel() > 0
        if meta._x.takes_partials(meta.recipe) and x2.numel():
            x8 = quantize_bf16_partials(x2, meta.x_scale, "e4m3", meta._x.partials)
            out = mm_fp8_bias(x8, meta.w_cached[2], meta.x_scale, meta.w_scale,
                              bias if has_bias else None).reshape(*x.shape[:-1], w.size(0))
            meta._x.push_partials(meta.recipe, fmt)
            return out
        x8, amax_x = quantize_bf16(x2, meta.x_scale, "e4m3")
        out = mm_fp8_bias(x8, meta.w_cached[2], meta.x_scale, meta.w_scale,
                          bias if has_bias else None).reshape(*x.shape[:-1], w.size(0))
        meta.update_x(amax_x, fmt)
        return out
    if meta._x.takes_partials(meta.recipe) and meta._w.takes_partials(meta.recipe) and x.numel() and w.numel():
        # the fused forward's arithmetic (both operands quantized with the rings' current steps,
        # GEMM with the bias in its epilogue), the two amax values going to their rings as
        # per-workgroup maxima
        x2 = x.reshape(-1, w.size(1))
        has_bias = bias is not None and bias.numel() > 0
        x8 = quantize_bf16_partials(x2, meta.x_scale, "e4m3", meta._x.partials)
        w8 = quantize_bf16_partials(w, meta.w_scale, "e4m3", meta._w.partials)
        out = mm_fp8_bias(x8, w8, meta.x_scale, meta.w_scale,
                          bias if has_bias else None).reshape(*x.shape[:-1], w.size(0))
        meta._x.push_partials(meta.recipe, fmt)
        meta._w.push_partials(meta.recipe, fmt)
        meta.note_w_push(w)
        return out
    out, amax_x, amax_w = linear_forward_fp8(x, w, bias, meta.x_scale, meta.w_scale)
    meta.update_x(amax_x, fmt)
    meta.update_w(amax_w, fmt)
    meta.note_w_push(w)
    return out


def fp8_linear_backward(g: torch.Tensor, x: torch.Tensor, w: torch.Tensor, masks):
    """Scaled fp8 linear backward (fp8.py:308-330): gradient quantized once in the
    backward format, dX and dW GEMMs share it."""
    st = fp8_state()
    fmt = st.fp8_format.bwd()
    meta = st.get_weight_meta(w)
    dynamic = isinstance(st.recipe, DynamicScaling)
    if dynamic:
        sg = _dynamic_scale(g, st.recipe, fmt)
        sw = _dynamic_scale(w, st.recipe, fmt)
        sx = _dynamic_scale(x, st.recipe, fmt)
    else:
        if not meta.g_init:
            meta.init_g(g, fmt)
        sg, sw, sx = meta.g_scale, meta.w_scale, meta.x_scale
    gx, gw, gb, amax_g = linear_backward_fp8(g, x, w, masks, sg, sw, sx, fmt)
    if not dynamic:
        meta.update_g(amax_g, fmt)
    return gx, gw, gb


def fp8_linear_enable(enabled: bool = True) -> None:
    fp8_state().enabled = enabled


def fp8_cache_weights(enabled: Optional[bool] = True) -> None:
    """Keep each weight's fp8 codes between forwards while the weight is unmodified
    (inference, or several micro-batches per optimizer step): True / False force it on
    or off for every Linear, None restores the default, which caches exactly where
    autograd is off or the weight takes no gradient. The reference quantizes the weight
    in every call (fp8.py:291-299); outputs and scaling state do not differ."""
    st = fp8_state()
    st.cache_weights = enabled
    if enabled is False:
        st._dyn_w.clear()
        for meta in st._metas.values():
            meta.w_cached = None


def fp8_linear_enabled() -> bool:
    return fp8_state().enabled


def _fp8_supported(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Only the contraction must line up; ragged M / N are handled by the kernels
    (fp8.py:348-356)."""
    return x.dim() >= 2 and w.dim() == 2 and x.size(-1) == w.size(1)


def _fp8_handler(x, w, bias):
    if (
        fp8_linear_enabled()
        and x.dtype == torch.bfloat16
        and w.dtype == torch.bfloat16
        and _fp8_supported(x, w)
    ):
        return fp8_linear_forward(x, w, bias)
    return None


def _fp8_backward_handler(input_tensor, grad_output, weight, output_mask):
    if (
        fp8_linear_enabled()
        and weight.dtype == torch.bfloat16
        and _fp8_supported(grad_output, weight)
    ):
        return fp8_linear_backward(grad_output, input_tensor, weight, list(output_mask))
    return None


# importing this module installs the aten::linear override (fp8.py:404-406)
dispatch.register_handler(_fp8_handler, _fp8_backward_handler)
