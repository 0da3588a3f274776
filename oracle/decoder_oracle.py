"""CPU restatement of the reference decoder forward with every Linear computed by
the W8A8 oracle. TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Works on a plain ``state_dict`` (parameter names of astrai/model/transformer.py:43-62)
so that it shares no code with the product's modules. Arithmetic followed:
  embed -> blocks -> final RMSNorm -> lm_head over all tokens   transformer.py:126-146
  x = attn(input_norm(x)) + x ; x = mlp(post_attention_norm(x)) + x   decoder_block.py:59-70
  q/k/v projections, rotary on q and k, SDPA, o_proj             components/attention.py:69-84
  rotary = complex multiply of adjacent pairs in fp32, cast back extension/backend/rotary.py:25-33
  cos/sin tables, angles in fp64                                  components/rope.py:8-24
  KV heads expanded by repeating each head n_rep times            extension/backend/attention.py:244-253
  causal SDPA                                                     extension/backend/attention.py:443-470
  MLP = down(up(x) * silu(gate(x)))                               components/mlp.py:40-43
  RMSNorm = F.rms_norm                                            components/norm.py:14-15
"""

from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
import torch.nn.functional as F

from oracle import w8a8_oracle as O


def rotary_table(dim: int, max_len: int, base: float) -> torch.Tensor:
    theta = base ** (-torch.arange(0, dim, 2, dtype=torch.float64) / dim)
    t = torch.arange(0, max_len, dtype=torch.float64)
    freqs = torch.outer(t, theta).float()
    return torch.stack([torch.cos(freqs), torch.sin(freqs)], dim=-1)


def rotary_base_of(cfg) -> float:
    """Base of the rotary table of a config: ``rope_theta`` (10000 when None,
    astrai/model/transformer.py:41), times ``factor ** (dim / (dim - 2))`` under NTK
    ``rope_scaling`` (astrai/model/components/rope.py:27-28,44-50; "ntk" is the default
    type, other types change nothing there)."""
    dim = cfg.hidden_size // cfg.num_attention_heads
    base = 10000.0 if cfg.rope_theta is None else float(cfg.rope_theta)
    scaling = getattr(cfg, "rope_scaling", None)
    if scaling is not None and scaling.get("type", "ntk") == "ntk":
        base = base * float(scaling.get("factor", 1.0)) ** (dim / (dim - 2))
    return base


def apply_rotary(x: torch.Tensor, freqs_cis: torch.Tensor) -> torch.Tensor:
    cos, sin = freqs_cis[..., 0], freqs_cis[..., 1]
    xc = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
    rot = xc * torch.complex(cos, sin).unsqueeze(-2)
    return torch.view_as_real(rot).flatten(-2).to(x.dtype)


def rope_cache_write(qkv: torch.Tensor, freqs_cis: torch.Tensor, positions: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: torch.Tensor, n_heads: int, n_kv_heads: int,
                     head_dim: int) -> torch.Tensor:
    """What sits between the q/k/v projections and the attention call with a cache
    (components/attention.py:19-85): split ``qkv [B, S, (H + 2 H_kv) D]``, rotate q and k
    (:func:`apply_rotary`), permute to ``[B, heads, S, D]``, write k and v into the caches
    ``[B, H_kv, max_len, D]`` at ``positions [S]`` (in place) and return q."""
    b, s, _ = qkv.shape
    nq, nkv = n_heads * head_dim, n_kv_heads * head_dim
    q = qkv[..., :nq].reshape(b, s, n_heads, head_dim)
    k = qkv[..., nq:nq + nkv].reshape(b, s, n_kv_heads, head_dim)
    v = qkv[..., nq + nkv:].reshape(b, s, n_kv_heads, head_dim)
    q, k = apply_rotary(q, freqs_cis), apply_rotary(k, freqs_cis)
    k_cache.index_copy_(2, positions, k.permute(0, 2, 1, 3))
    v_cache.index_copy_(2, positions, v.permute(0, 2, 1, 3))
    return q.permute(0, 2, 1, 3).contiguous()


def attn_cached(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                positions: torch.Tensor) -> torch.Tensor:
    """Attention of ``q [B, H, S, D]`` over the caches ``[B, H_kv, max_len, D]`` where token ``s``
    sees keys ``0..positions[s]``: head expansion (extension/backend/attention.py:244-253) and
    ``softmax(q k^T / sqrt(D)) v`` in float32 (:443-498), returned token-major ``[B, S, H*D]`` in
    the input dtype, as the cached branch of components/attention.py:19-85 hands it to ``o_proj``."""
    b, h, s, d = q.shape
    n_rep = h // k_cache.size(1)
    # repeat_kv works on [B, S, H_kv, D]; the caches are [B, H_kv, max_len, D]
    k = repeat_kv(k_cache.transpose(1, 2), n_rep).transpose(1, 2).float()
    v = repeat_kv(v_cache.transpose(1, 2), n_rep).transpose(1, 2).float()
    scores = q.float() @ k.transpose(-1, -2) / (d ** 0.5)          # [B, H, S, max_len]
    key_pos = torch.arange(k_cache.size(2))
    visible = key_pos[None, :] <= positions[:, None]                 # [S, max_len]
    scores = scores.masked_fill(~visible[None, None], float("-inf"))
    out = torch.softmax(scores, dim=-1) @ v                          # [B, H, S, D]
    return out.permute(0, 2, 1, 3).reshape(b, s, h * d).to(q.dtype)


def attn_paged_decode(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                      kv_indptr: torch.Tensor, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Decode attention over a token-granular paged cache: ``q [B, H, D]``, pools
    ``[slots, H_kv, D]``; key ``j`` of sequence ``b`` is pool row
    ``req_to_token[req_pool_indices[b], j]`` for ``j < kv_indptr[b+1] - kv_indptr[b]``
    (csrc/kernels/attention/layout_policies.cuh:174-232; astrai/extension/ops/attention.py:93-147).
    A negative row ("empty padding") is not fetched -- its key and value are zeros -- but the
    position stays in the attended range [0, kv_len): the reference gates the load on the slot
    (layout_policies.cuh:104-110,212-219; decode_split_kv_mma.cuh:75-82) and masks by position
    only (decode_split_kv_mma.cuh:107-110), so such a position enters the softmax with score 0.
    ``mask`` (bool ``[B, width]``, indexed by sequence and position, True = attend) hides
    positions on top of that (csrc/kernels/attention/entry_utils.cuh:226-237,
    mma_utils.cuh:196-199); the reference reads past a mask narrower than a sequence, here such
    positions are hidden. ``softmax(q k^T / sqrt(D)) v`` in float32 per sequence; a sequence
    without a visible key gives zeros (mma_utils.cuh:217-218, the guarded 1/l of the kernels).
    Returns ``[B, H, D]`` in the input dtype."""
    b, h, d = q.shape
    n_rep = h // k_pool.size(1)
    out = torch.zeros(b, h, d, dtype=torch.float32)
    for i in range(b):
        n = int(kv_indptr[i + 1]) - int(kv_indptr[i])
        rows = req_to_token[int(req_pool_indices[i]), :n].long()
        if rows.numel() == 0:
            continue
        live = (rows >= 0)[:, None, None]
        k = torch.where(live, k_pool[rows.clamp_min(0)].float(), torch.zeros(())).repeat_interleave(n_rep, dim=1)
        v = torch.where(live, v_pool[rows.clamp_min(0)].float(), torch.zeros(())).repeat_interleave(n_rep, dim=1)
        scores = torch.einsum("hd,nhd->hn", q[i].float(), k) / (d ** 0.5)
        if mask is not None:
            seen = torch.zeros(n, dtype=torch.bool)
            w = min(n, mask.size(1))
            seen[:w] = mask[i, :w]
            if not bool(seen.any()):
                continue
            scores = scores.masked_fill(~seen[None], float("-inf"))
        out[i] = torch.einsum("hn,nhd->hd", torch.softmax(scores, dim=-1), v)
    return out.to(q.dtype)


def attn_paged_prefill(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                       req_to_token: torch.Tensor, req_pool_indices: torch.Tensor,
                       kv_indptr: torch.Tensor, qo_indptr: torch.Tensor,
                       causal: bool = True, mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Ragged prefill over the paged cache: packed ``q [total_q, H, D]``; sequence ``b`` owns
    rows ``qo_indptr[b] .. qo_indptr[b+1]`` and keys ``req_to_token[req_pool_indices[b], :kv_len]``;
    with ``causal`` row ``i`` of it sees keys ``0 .. kv_len - q_len + i``
    (csrc/kernels/attention/layout_policies.cuh:67-93,174-232). A negative pool row reads as a
    zero key and a zero value and is attended like any other position (the load is gated on the
    slot, the mask on the position: prefill_split_q_mma.cuh:84-89,121-124). ``mask`` (bool, True
    = attend): ``[B, kv]``, or ``[B, 1 | H, rows, kv]`` with ``rows`` 1 (every row) or counted
    inside each sequence, combined with the causal range by "and" (entry_utils.cuh:326-346,
    mma_utils.cuh:190-199); the reference reads past a mask with fewer rows or positions than
    a sequence, here those are hidden. float32 softmax attention per sequence; a row that sees
    no position gives zeros. Returns ``[total_q, H, D]`` in the input dtype."""
    total_q, h, d = q.shape
    n_rep = h // k_pool.size(1)
    out = torch.zeros(total_q, h, d, dtype=torch.float32)
    for b in range(req_pool_indices.numel()):
        q0, q1 = int(qo_indptr[b]), int(qo_indptr[b + 1])
        n = int(kv_indptr[b + 1]) - int(kv_indptr[b])
        if q1 == q0 or n == 0:
            continue
        rows = req_to_token[int(req_pool_indices[b]), :n].long()
        live = (rows >= 0)[:, None, None]
        k = torch.where(live, k_pool[rows.clamp_min(0)].float(), torch.zeros(())).repeat_interleave(n_rep, dim=1)
        v = torch.where(live, v_pool[rows.clamp_min(0)].float(), torch.zeros(())).repeat_interleave(n_rep, dim=1)
        scores = torch.einsum("qhd,nhd->hqn", q[q0:q1].float(), k) / (d ** 0.5)
        visible = torch.ones(q1 - q0, n, dtype=torch.bool)
        if causal:
            newest = (n - (q1 - q0)) + torch.arange(q1 - q0)
            visible &= torch.arange(n)[None, :] <= newest[:, None]
        visible = visible[None].expand(h, -1, -1)
        if mask is not None:
            m4 = mask[b][None, None, :] if mask.dim() == 2 else mask[b]      # [1 | H, rows, kv]
            cover = torch.zeros(m4.size(0), q1 - q0, n, dtype=torch.bool)
            w = min(n, m4.size(-1))
            if m4.size(1) == 1:
                cover[:, :, :w] = m4[:, :, :w]
            else:
                r = min(q1 - q0, m4.size(1))
                cover[:, :r, :w] = m4[:, :r, :w]
            visible = visible & cover
        scores = scores.masked_fill(~visible, float("-inf"))
        p = torch.softmax(scores, dim=-1)
        p = torch.where(visible.any(-1)[:, :, None], p, torch.zeros_like(p))
        out[q0:q1] = torch.einsum("hqn,nhd->qhd", p, v)
    return out.to(q.dtype)


def attn_dense(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: Optional[torch.Tensor] = None,
               causal_offset: int = -1, layout: int = 1) -> torch.Tensor:
    """The reference's dense kernels attn_decode / attn_prefill as one formula: ``q``, ``k``,
    ``v`` in layout 1 ``[B, L, H, D]`` or 0 ``[B, H, L, D]``; query head ``h`` reads KV head
    ``h // n_rep``; with ``causal_offset >= 0`` row ``i`` sees keys ``j <= i + causal_offset``
    (csrc/kernels/attention/prefill_split_q_mma.cuh:121-124; for the one row of a decode
    call that is layout_policies.cuh:138-141); ``mask`` (bool, True = attend) is ``[B, kv]``,
    ``[B, 1 | q, kv]`` or ``[B, 1 | H, 1 | q, kv]`` (entry_utils.cuh:56-86), "and"-ed with the
    causal range (mma_utils.cuh:196-199). float32 ``softmax(q k^T / sqrt(D)) v``; a row that
    sees nothing gives zeros. Returns ``q``'s shape and dtype."""
    if layout == 1:
        q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    b, h, lq, d = q.shape
    n_rep, lk = h // k.size(1), k.size(2)
    kf = k.float().repeat_interleave(n_rep, dim=1)
    vf = v.float().repeat_interleave(n_rep, dim=1)
    scores = q.float() @ kf.transpose(-1, -2) / (d ** 0.5)             # [B, H, lq, lk]
    visible = torch.ones(b, h, lq, lk, dtype=torch.bool)
    if causal_offset >= 0:
        visible &= (torch.arange(lk)[None, :] <= torch.arange(lq)[:, None] + causal_offset)[None, None]
    if mask is not None:
        m = mask
        if m.dim() == 2:
            m = m[:, None, None, :]
        elif m.dim() == 3:
            m = m[:, None]
        visible = visible & m
    scores = scores.masked_fill(~visible, float("-inf"))
    p = torch.softmax(scores, dim=-1)
    p = torch.where(visible.any(-1, keepdim=True), p, torch.zeros_like(p))
    out = (p @ vf).to(q.dtype)
    return out.transpose(1, 2) if layout == 1 else out


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    # x: [B, S, H_kv, D] -> [B, S, H_kv*n_rep, D]
    if n_rep == 1:
        return x
    h, d = x.shape[-2:]
    return x.unsqueeze(-2).expand(*x.shape[:-2], h, n_rep, d).reshape(*x.shape[:-2], h * n_rep, d)


def int8_linear_fn(sd: Dict[str, torch.Tensor], fast: bool = False) -> Callable[[torch.Tensor, str], torch.Tensor]:
    """Quantize every 2-D projection weight per output channel once; activations per token per call.
    ``fast``: the library int8 routine with its sampled self-check (timing legs only)."""
    q = {k: O.int8_quantize_rows(v) for k, v in sd.items()
         if v.dim() == 2 and not k.startswith("embed_tokens")}

    def lin(x: torch.Tensor, name: str) -> torch.Tensor:
        wq, sw = q[name]
        return O.int8_linear(x, wq, sw, fast=fast)

    return lin


def bf16_linear_fn(sd: Dict[str, torch.Tensor]) -> Callable[[torch.Tensor, str], torch.Tensor]:
    return lambda x, name: F.linear(x, sd[name])


def forward(sd: Dict[str, torch.Tensor], cfg, input_ids: torch.Tensor,
            lin: Callable[[torch.Tensor, str], torch.Tensor]) -> torch.Tensor:
    """Causal forward over ``input_ids [B, S]``; returns logits ``[B, S, vocab]`` (bf16)."""
    b, s = input_ids.shape
    nh, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    hd = cfg.hidden_size // nh
    x = F.embedding(input_ids, sd["embed_tokens.weight"])
    fc = rotary_table(hd, s, rotary_base_of(cfg)).unsqueeze(0)  # [1, S, hd/2, 2]
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        h = F.rms_norm(x, (cfg.hidden_size,), sd[p + "input_norm.weight"], cfg.rms_norm_eps)
        q = lin(h, p + "attention.q_proj.weight").reshape(b, s, nh, hd)
        k = lin(h, p + "attention.k_proj.weight").reshape(b, s, nkv, hd)
        v = lin(h, p + "attention.v_proj.weight").reshape(b, s, nkv, hd)
        q, k = apply_rotary(q, fc), apply_rotary(k, fc)
        k, v = repeat_kv(k, nh // nkv), repeat_kv(v, nh // nkv)
        a = F.scaled_dot_product_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3),
                                           v.permute(0, 2, 1, 3), is_causal=True)
        a = a.permute(0, 2, 1, 3).reshape(b, s, cfg.hidden_size)
        x = lin(a, p + "attention.o_proj.weight") + x
        h = F.rms_norm(x, (cfg.hidden_size,), sd[p + "post_attention_norm.weight"], cfg.rms_norm_eps)
        up = lin(h, p + "mlp.up.weight")
        gate = lin(h, p + "mlp.gate.weight")
        x = lin(up * F.silu(gate), p + "mlp.down.weight") + x
    hidden = F.rms_norm(x, (cfg.hidden_size,), sd["norm.weight"], cfg.rms_norm_eps)
    return lin(hidden, "lm_head.weight")


def forward_cached(sd: Dict[str, torch.Tensor], cfg, input_ids: torch.Tensor,
                   lin: Callable[[torch.Tensor, str], torch.Tensor], k_cache: torch.Tensor,
                   v_cache: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """The same forward for a block of tokens at ``positions [S]`` with a dense KV cache
    ``[layers, B, H_kv, max_len, D]`` (updated in place): the cached branch of
    components/attention.py:19-85, i.e. :func:`rope_cache_write` then :func:`attn_cached` per
    layer. A prefill followed by one-token calls reproduces :func:`forward` (the contract of
    tests/module/test_model_forward.py:71-115)."""
    b, s = input_ids.shape
    nh, nkv = cfg.num_attention_heads, cfg.num_key_value_heads
    hd = cfg.hidden_size // nh
    x = F.embedding(input_ids, sd["embed_tokens.weight"])
    table = rotary_table(hd, int(positions.max()) + 1, rotary_base_of(cfg))
    fc = table.index_select(0, positions).unsqueeze(0)      # [1, S, hd/2, 2]
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        h = F.rms_norm(x, (cfg.hidden_size,), sd[p + "input_norm.weight"], cfg.rms_norm_eps)
        qkv = torch.cat([lin(h, p + "attention.q_proj.weight"), lin(h, p + "attention.k_proj.weight"),
                         lin(h, p + "attention.v_proj.weight")], dim=-1)
        q = rope_cache_write(qkv, fc, positions, k_cache[i], v_cache[i], nh, nkv, hd)
        a = attn_cached(q, k_cache[i], v_cache[i], positions)
        x = lin(a, p + "attention.o_proj.weight") + x
        h = F.rms_norm(x, (cfg.hidden_size,), sd[p + "post_attention_norm.weight"], cfg.rms_norm_eps)
        up = lin(h, p + "mlp.up.weight")
        gate = lin(h, p + "mlp.gate.weight")
        x = lin(up * F.silu(gate), p + "mlp.down.weight") + x
    hidden = F.rms_norm(x, (cfg.hidden_size,), sd["norm.weight"], cfg.rms_norm_eps)
    return lin(hidden, "lm_head.weight")

