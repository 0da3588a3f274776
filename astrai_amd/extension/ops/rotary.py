"""Rotary embedding entry point with the call surface of the reference's
``astrai/extension/ops/rotary.py`` (lines 24-39): ``x`` packed ``[tokens, heads, head_dim]``
or dense ``[batch, seq_len, heads, head_dim]`` in bf16, ``freqs_cis`` fp32 with the same token
axes followed by ``[head_dim/2, 2]``. Inputs that are not contiguous are copied first, as
there; a missing kernel raises."""

from __future__ import annotations

from torch import Tensor

from astrai_amd.extension import loader


def rotary_emb(x: Tensor, freqs_cis: Tensor) -> Tensor:
    entry = loader.get_module("rotary_emb") if loader.is_available("rotary_emb") else None
    if entry is None:
        raise RuntimeError("kernel 'rotary_emb' is not available: libastrai_w8a8.so did not load "
                           "(build it with `make -C astrai_amd/csrc`)")
    return entry.rotary_emb(x if x.is_contiguous() else x.contiguous(),
                            freqs_cis if freqs_cis.is_contiguous() else freqs_cis.contiguous())
