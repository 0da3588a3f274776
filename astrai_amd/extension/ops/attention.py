"""Attention entry points with the call surface of the reference's
``astrai/extension/ops/attention.py``: one function per registered kernel, boolean
``is_causal`` instead of the kernels' ``causal_offset``.

How ``is_causal`` turns into an offset there, kept here:

======================  =============================  ==========
function                offset when ``is_causal``      lines
======================  =============================  ==========
``attn_decode``         ``kv_len - 1``                 41-64
``attn_prefill``        ``kv_len - q_len``             67-90
``attn_paged_decode``   ``0`` (any value >= 0 works)   93-147
``attn_paged_prefill``  ``0``                          150-207
======================  =============================  ==========

and ``-1`` (no causal limit) otherwise. The dense functions take ``[batch, seq_len,
heads, head_dim]`` tensors, the paged ones packed queries and flat pools. Nothing here
computes: a missing kernel raises, as in the reference (its lines 33-38).
"""

from __future__ import annotations

import enum
from typing import Optional

from torch import Tensor

from astrai_amd.extension import loader


class TensorLayout(enum.IntEnum):
    """Layout codes of the dense kernels (the reference's enum of the same name)."""

    BHLD = 0  # [batch, n_heads, seq_len, head_dim]
    BLHD = 1  # [batch, seq_len, n_heads, head_dim]


def _kernel(name: str):
    entry = loader.get_module(name) if loader.is_available(name) else None
    if entry is None:
        raise RuntimeError(f"kernel '{name}' is not available: libastrai_w8a8.so did not load "
                           "(build it with `make -C astrai_amd/csrc`)")
    return getattr(entry, name)


def _offset(is_causal: bool, when_causal: int) -> int:
    return when_causal if is_causal else -1


def attn_decode(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None,
                is_causal: bool = False) -> Tensor:
    """One query token per sequence: ``q [batch, 1, heads, 128]`` against ``k``, ``v``
    ``[batch, kv_len, kv_heads, 128]`` (bf16); ``mask`` bool ``[batch, kv_len]`` or
    ``[batch, 1, kv_len]``, True = attend. Returns ``q``'s shape."""
    return _kernel("attn_decode")(q, k, v, mask=mask, causal_offset=_offset(is_causal, k.size(1) - 1),
                                  layout=int(TensorLayout.BLHD))


def attn_prefill(q: Tensor, k: Tensor, v: Tensor, mask: Optional[Tensor] = None,
                 is_causal: bool = False) -> Tensor:
    """A block of query rows per sequence: ``q [batch, q_len, heads, 128]`` against ``k``, ``v``
    ``[batch, kv_len, kv_heads, 128]``; with ``is_causal`` the last row sees every key. ``mask``
    bool ``[batch, kv_len]`` or ``[batch, q_len, kv_len]``. Returns ``q``'s shape."""
    return _kernel("attn_prefill")(q, k, v, mask=mask,
                                   causal_offset=_offset(is_causal, k.size(1) - q.size(1)),
                                   layout=int(TensorLayout.BLHD))


def attn_paged_decode(q: Tensor, k_cache: Tensor, v_cache: Tensor, req_to_token: Tensor,
                      req_pool_indices: Tensor, kv_indptr: Tensor, new_k: Optional[Tensor] = None,
                      new_v: Optional[Tensor] = None, mask: Optional[Tensor] = None,
                      is_causal: bool = False, o_part_buf: Optional[Tensor] = None,
                      ml_part_buf: Optional[Tensor] = None, out_buf: Optional[Tensor] = None) -> Tensor:
    """Decode over the flat pool: ``q [batch, heads, 128]``, pools ``[slots, kv_heads, 128]``,
    ``req_to_token`` / ``req_pool_indices`` / ``kv_indptr`` int32; ``new_k`` / ``new_v`` are stored
    at each sequence's newest position first; ``mask`` bool ``[batch, positions]``; ``out_buf``
    receives the result when given. Returns ``[batch, heads, 128]``."""
    return _kernel("attn_paged_decode")(q, k_cache, v_cache, req_to_token, req_pool_indices, kv_indptr,
                                        new_k=new_k, new_v=new_v, mask=mask,
                                        causal_offset=_offset(is_causal, 0), o_part_buf=o_part_buf,
                                        ml_part_buf=ml_part_buf, out_buf=out_buf)


def attn_paged_prefill(q: Tensor, k_cache: Tensor, v_cache: Tensor, req_to_token: Tensor,
                       req_pool_indices: Tensor, kv_indptr: Tensor, qo_indptr: Tensor,
                       q_tile_to_batch: Tensor, q_tile_to_index: Tensor, mask: Optional[Tensor] = None,
                       is_causal: bool = False) -> Tensor:
    """Ragged prefill over the flat pool: packed ``q [total_q, heads, 128]``, per-sequence row
    ranges ``qo_indptr`` and key counts ``kv_indptr``, the 64-row tile schedule, ``mask`` bool
    ``[batch, kv]`` or ``[batch, 1 | heads, rows, kv]``. Returns ``[total_q, heads, 128]``."""
    return _kernel("attn_paged_prefill")(q, k_cache, v_cache, req_to_token, req_pool_indices, kv_indptr,
                                         qo_indptr, q_tile_to_batch, q_tile_to_index, mask,
                                         causal_offset=_offset(is_causal, 0))
