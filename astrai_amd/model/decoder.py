"""Dense decoder whose every projection is ``Linear -> F.linear``, so that the
``aten::linear`` hook of ``astrai_amd.extension`` routes it through the W8A8
kernels without the model knowing.

Module structure, parameter names, initialisation and arithmetic follow the
reference: ``AutoRegressiveLM`` (astrai/model/transformer.py:29-152),
``DecoderBlock`` (components/decoder_block.py:19-76), ``GQA``
(components/attention.py:19-85), ``MLP`` (components/mlp.py:32-43), ``Linear``
(components/linear.py:7-24), ``RMSNorm`` (components/norm.py:7-15), ``Embedding``
(components/embedding.py:9-26), rotary tables and their application
(components/rope.py:8-76, extension/backend/rotary.py:25-33), GQA head expansion
and causal SDPA (extension/backend/attention.py:244-253,443-470).

The reference's inference path packs requests and walks a paged cache per request
with host reads; here requests form a dense ``[batch, seq]`` block over a dense
``[layer, batch, kv_head, position, head_dim]`` cache, which is the same
arithmetic for equal-length prompts and keeps the decode step free of host
synchronisation, hence HIP-graph capturable.

``fuse_int8_weights(model)`` adds a second way through the same blocks for int8
inference: q|k|v and gate|up weights concatenated into one int8 matrix each, the
residual add + RMSNorm and the SwiGLU product fused with the per-token quantizer,
so a block issues 4 GEMMs and 4 producer kernels around its attention core
instead of 7 GEMMs, 7 quantizers, 2 norms, 2 adds and a product. The arithmetic
per element is that of the modular path (concatenating per-channel quantized rows
changes no row; the fused producers round where the separate ops round).
"""

from dataclasses import dataclass
from types import SimpleNamespace
from typing import Dict, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Tensor


@dataclass
class AutoRegressiveLMConfig:
    """The fields of the reference's config (config/model_config.py:38-101) that a
    dense GQA decoder uses."""

    vocab_size: int = 32000
    hidden_size: int = 2048
    num_hidden_layers: int = 24
    num_attention_heads: int = 16
    num_key_value_heads: int = 4
    intermediate_size: int = 5632
    rms_norm_eps: float = 1e-5
    rope_theta: Optional[float] = 10000.0
    rope_scaling: Optional[dict] = None   # e.g. {"type": "ntk", "factor": 4.0}
    max_position_embeddings: int = 2048
    tie_word_embeddings: bool = False


class Linear(nn.Module):
    def __init__(self, in_dim: int, out_dim: int, bias: bool = False, init_std: float = 0.02):
        super().__init__()
        self.weight = nn.Parameter(torch.empty((out_dim, in_dim)))
        self.bias = nn.Parameter(torch.zeros(out_dim)) if bias else None
        self.init_std = init_std

    def reset_parameters(self):
        nn.init.normal_(self.weight, mean=0.0, std=self.init_std)
        if self.bias is not None:
            bound = 1 / (self.weight.size(1) ** 0.5)
            nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, x: Tensor) -> Tensor:
        return F.linear(x, self.weight, self.bias)


class RMSNorm(nn.Module):
    def __init__(self, dim: int, norm_eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.normalized_shape = (dim,)
        self.norm_eps = norm_eps

    def forward(self, x: Tensor) -> Tensor:
        return F.rms_norm(x, self.normalized_shape, self.weight, self.norm_eps)


class Embedding(nn.Module):
    def __init__(self, vocab_size: int, embedding_dim: int):
        super().__init__()
        self.weight = nn.Parameter(torch.empty((vocab_size, embedding_dim)))

    def reset_parameters(self):
        nn.init.normal_(self.weight, mean=0.0, std=0.02)

    def forward(self, x: Tensor) -> Tensor:
        return F.embedding(x, self.weight)


def get_rotary_emb(dim: int, max_len: int, base: float = 10000.0) -> Tensor:
    """``[max_len, dim/2, 2]`` fp32 table of (cos, sin), angles computed in fp64."""
    theta = base ** (-torch.arange(0, dim, 2, dtype=torch.float64) / dim)
    t = torch.arange(0, max_len, dtype=torch.float64)
    freqs = torch.outer(t, theta).float()
    return torch.stack([torch.cos(freqs), torch.sin(freqs)], dim=-1)


def ntk_base(base: float, dim: int, factor: float) -> float:
    """NTK-aware stretching of the rotary base (components/rope.py:27-28)."""
    return base * (factor ** (dim / (dim - 2)))


def rotary_base(rope_theta: Optional[float], dim: int, rope_scaling: Optional[dict]) -> float:
    """The base the rotary table is built from: ``rope_theta`` (10000 when absent,
    transformer.py:41), stretched by :func:`ntk_base` when ``rope_scaling`` names the
    type "ntk" (the default type); any other type leaves the base alone, as the
    reference's ``RotaryEmbedding.__init__`` does (components/rope.py:44-50)."""
    base = 10000.0 if rope_theta is None else rope_theta
    if rope_scaling is not None and rope_scaling.get("type", "ntk") == "ntk":
        base = ntk_base(base, dim, rope_scaling.get("factor", 1.0))
    return base


def apply_rotary_emb(x: Tensor, freqs_cis: Tensor) -> Tensor:
    """Rotate adjacent (even, odd) pairs of the head dimension; fp32 math, cast back.
    ``x`` is ``[batch, seq, heads, head_dim]``, ``freqs_cis`` ``[batch|1, seq, head_dim/2, 2]``."""
    cos, sin = freqs_cis[..., 0].unsqueeze(-2), freqs_cis[..., 1].unsqueeze(-2)
    x_ = x.float().reshape(*x.shape[:-1], -1, 2)
    xe, xo = x_[..., 0], x_[..., 1]
    out = torch.stack([xe * cos - xo * sin, xe * sin + xo * cos], dim=-1)
    return out.flatten(-2).to(x.dtype)


def repeat_kv(x: Tensor, n_rep: int) -> Tensor:
    """``[B, H_kv, S, D] -> [B, H_kv*n_rep, S, D]``, each KV head repeated n_rep times in place order."""
    if n_rep == 1:
        return x
    b, h, s, d = x.shape
    return x.unsqueeze(2).expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


class DenseKVCache:
    """``k``/``v``: ``[layers, batch, kv_heads, max_len, head_dim]``."""

    def __init__(self, config: AutoRegressiveLMConfig, batch: int, max_len: int, device, dtype):
        hd = config.hidden_size // config.num_attention_heads
        shape = (config.num_hidden_layers, batch, config.num_key_value_heads, max_len, hd)
        self.k = torch.zeros(shape, device=device, dtype=dtype)
        self.v = torch.zeros(shape, device=device, dtype=dtype)
        self.max_len = max_len


class GQA(nn.Module):
    def __init__(self, dim: int, n_heads: int, n_kv_heads: int, layer_id: int, n_layers: int):
        super().__init__()
        assert dim % n_heads == 0 and n_heads % n_kv_heads == 0
        self.head_dim = dim // n_heads
        self.layer_id = layer_id
        self.dim, self.n_heads, self.n_kv_heads = dim, n_heads, n_kv_heads
        self.n_rep = n_heads // n_kv_heads
        self.q_proj = Linear(dim, n_heads * self.head_dim)
        self.k_proj = Linear(dim, n_kv_heads * self.head_dim)
        self.v_proj = Linear(dim, n_kv_heads * self.head_dim)
        self.o_proj = Linear(dim, dim, init_std=0.02 / (2 * n_layers) ** 0.5)

    def forward(self, x: Tensor, rotary_emb: Tensor, kv_cache: Optional[DenseKVCache],
                positions: Optional[Tensor], key_mask: Optional["_KeyMask"]) -> Tensor:
        out = self.core(self.q_proj(x), self.k_proj(x), self.v_proj(x), rotary_emb, kv_cache,
                        positions, key_mask)
        return self.o_proj(out)

    def core(self, q: Tensor, k: Tensor, v: Tensor, rotary_emb: Tensor,
             kv_cache: Optional[DenseKVCache], positions: Optional[Tensor],
             key_mask: Optional["_KeyMask"]) -> Tensor:
        """Everything between the q/k/v projections and ``o_proj``: ``[B, S, *]`` in,
        ``[B, S, dim]`` out."""
        b, s = q.shape[0], q.shape[1]
        q = q.reshape(b, s, self.n_heads, self.head_dim)
        k = k.reshape(b, s, self.n_kv_heads, self.head_dim)
        v = v.reshape(b, s, self.n_kv_heads, self.head_dim)
        q, k = apply_rotary_emb(q, rotary_emb), apply_rotary_emb(k, rotary_emb)
        q, k, v = q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)
        if kv_cache is None:
            out = F.scaled_dot_product_attention(q, repeat_kv(k, self.n_rep), repeat_kv(v, self.n_rep),
                                                 is_causal=True)
        else:
            # write the new keys / values at `positions` (a device index tensor: no
            # host read), then attend over the cache under `key_mask`
            kv_cache.k[self.layer_id].index_copy_(2, positions, k)
            kv_cache.v[self.layer_id].index_copy_(2, positions, v)
            # the n_rep query heads that share a KV head are folded into the query
            # axis ([B, H_kv, n_rep*S, D]) instead of copying the cache n_rep times:
            # the same dot products and softmax rows as after repeat_kv
            out = self._attend_cache(q, kv_cache, key_mask)
        return out.permute(0, 2, 1, 3).reshape(b, s, self.dim)

    def _attend_cache(self, q: Tensor, kv_cache: DenseKVCache, key_mask: "_KeyMask") -> Tensor:
        """``q [B, H, S, D]`` against the layer's cache under the block's mask (``key_mask.get()``:
        ``[1, 1, n_rep*S, max_len]``, one copy per query head of a KV group)."""
        b, _, s, _ = q.shape
        qf = q.reshape(b, self.n_kv_heads, self.n_rep * s, self.head_dim)
        out = F.scaled_dot_product_attention(qf, kv_cache.k[self.layer_id],
                                             kv_cache.v[self.layer_id], attn_mask=key_mask.get())
        return out.reshape(b, self.n_heads, s, self.head_dim)

    def core_fused_qkv(self, qkv: Tensor, rotary_emb: Tensor, kv_cache: DenseKVCache,
                       positions: Tensor, key_mask: "_KeyMask"):
        """Same as :meth:`core` for a fused ``q|k|v`` projection ``[B, S, (H + 2 H_kv) D]`` with a
        cache: rotation, permutes and the cache write are one kernel. Returns the attention
        output already quantized per token, ``(int8 [B*S, dim], fp32 [B*S, 1])``: for a few new
        tokens straight out of the split-context attention kernel (mask from ``positions``,
        token-major), for longer blocks the causal block kernel followed by the quantizer; other
        head_dim / groupings run the general paged kernel over the same cache (SDPA only for
        head layouts no kernel takes)."""
        from astrai_amd.extension import _cabi
        q = _cabi.rope_cache_write(qkv, rotary_emb[0], positions, kv_cache.k[self.layer_id],
                                   kv_cache.v[self.layer_id], self.n_heads, self.n_kv_heads,
                                   self.head_dim)
        return self.attend_rotated(q, kv_cache, positions, key_mask)

    def attend_rotated(self, q: Tensor, kv_cache: DenseKVCache, positions: Tensor, key_mask: "_KeyMask"):
        """The attention of :meth:`core_fused_qkv` for an already rotated ``q [B, H, S, D]``
        whose keys and values are in the cache."""
        from astrai_amd.extension import _cabi
        b, _, s, _ = q.shape
        if _cabi.attn_decode_supported(self.n_heads, self.n_kv_heads, s, self.head_dim):
            return _cabi.attn_decode(q, kv_cache.k[self.layer_id], kv_cache.v[self.layer_id], positions,
                                     quantized=True)
        if _cabi.attn_prefill_supported(self.n_heads, self.n_kv_heads, self.head_dim):
            # causal block kernel: no mask tensor, no head expansion, token-major output
            return _cabi.quantize_int8_rows(
                _cabi.attn_prefill(q, kv_cache.k[self.layer_id], kv_cache.v[self.layer_id], positions))
        if _cabi.attn_cache_rows_supported(self.n_heads, self.n_kv_heads, self.head_dim):
            # other head shapes: the general kernel over the same cache, addressed per KV head
            return _cabi.quantize_int8_rows(
                _cabi.attn_cache_rows(q, kv_cache.k[self.layer_id], kv_cache.v[self.layer_id], positions))
        out = self._attend_cache(q, kv_cache, key_mask)
        return _cabi.quantize_int8_rows(out.permute(0, 2, 1, 3).reshape(b, s, self.dim))


class _KeyMask:
    """The mask of a block of new tokens against the cache, ``key position <= token position``,
    built on first use and shared by the layers of one forward: the HIP attention kernels take
    ``positions`` themselves, so a model on those never builds it (three small launches a step)."""

    def __init__(self, positions: Tensor, max_len: int, n_rep: int):
        self.positions, self.max_len, self.n_rep = positions, max_len, n_rep
        self._mask: Optional[Tensor] = None

    def get(self) -> Tensor:
        if self._mask is None:
            key_pos = torch.arange(self.max_len, device=self.positions.device)
            mask = (key_pos[None, :] <= self.positions[:, None])[None, None]  # [1,1,seq,max_len]
            if self.n_rep > 1:  # one copy per query head of a KV group, made once for all layers
                mask = mask.repeat(1, 1, self.n_rep, 1)
            self._mask = mask
        return self._mask


class MLP(nn.Module):
    def __init__(self, dim: int, dim_ffn: int, down_init_std: float = 0.02):
        super().__init__()
        self.up = Linear(dim, dim_ffn)
        self.gate = Linear(dim, dim_ffn)
        self.down = Linear(dim_ffn, dim, init_std=down_init_std)

    def forward(self, x: Tensor) -> Tensor:
        return self.down(self.up(x) * F.silu(self.gate(x)))


class DecoderBlock(nn.Module):
    def __init__(self, config: AutoRegressiveLMConfig, layer_id: int):
        super().__init__()
        n = config.num_hidden_layers
        self.attention = GQA(config.hidden_size, config.num_attention_heads,
                             config.num_key_value_heads, layer_id, n)
        self.input_norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.post_attention_norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.mlp = MLP(config.hidden_size, config.intermediate_size,
                       down_init_std=0.02 / (2 * n) ** 0.5)

        self.fused_int8 = None  # set by fuse_int8_weights

    def forward(self, x, rotary_emb, kv_cache, positions, key_mask):
        if self.fused_int8 is not None and _fused_int8_active(x):
            return self._forward_fused_int8(x, rotary_emb, kv_cache, positions, key_mask)
        x = self.attention(self.input_norm(x), rotary_emb, kv_cache, positions, key_mask) + x
        return self.mlp(self.post_attention_norm(x)) + x

    def _forward_fused_int8(self, x, rotary_emb, kv_cache, positions, key_mask):
        """The block on int8 projections with fused producers and epilogues: each norm is one
        kernel with the per-token quantizer, and the output and down projections add the
        residual stream in their epilogues (``attn_output + x``, ``mlp_output + x``)."""
        # (the C-ABI wrappers directly: a dispatcher round trip per call is what an eager decode step,
        # ~220 launches of a few microseconds each, would otherwise spend most of its time in)
        from astrai_amd.extension import _cabi
        f, att = self.fused_int8, self.attention
        b, s, d = x.shape
        xq, sx, _, _ = _cabi.add_rmsnorm_quantize_int8(x, self.input_norm.weight, self.input_norm.norm_eps)
        if kv_cache is None:
            qkv = _cabi.mm_int8(xq, f.wqkv, sx, f.sqkv).reshape(b, s, -1)
            nq, nkv = att.n_heads * att.head_dim, att.n_kv_heads * att.head_dim
            aq, sa = _cabi.quantize_int8_rows(
                att.core(qkv[..., :nq], qkv[..., nq:nq + nkv], qkv[..., nq + nkv:], rotary_emb, None,
                         positions, key_mask))
        elif _cabi.mm_int8_rope_cache_supported(b * s, d, att.head_dim, f.wqkv.size(0), b, att.n_heads,
                                                att.n_kv_heads, kv_cache.max_len):
            # a few new tokens, or a long block at head_dim 128: the projection's epilogue rotates q
            # and k and writes the cache
            q = _cabi.mm_int8_rope_cache(xq, f.wqkv, sx, f.sqkv, rotary_emb[0], positions,
                                         kv_cache.k[att.layer_id], kv_cache.v[att.layer_id],
                                         b, s, att.n_heads, att.n_kv_heads, att.head_dim)
            aq, sa = att.attend_rotated(q, kv_cache, positions, key_mask)
        else:
            qkv = _cabi.mm_int8(xq, f.wqkv, sx, f.sqkv).reshape(b, s, -1)
            aq, sa = att.core_fused_qkv(qkv, rotary_emb, kv_cache, positions, key_mask)
        h = _cabi.mm_int8_resid(aq, f.wo, sa, f.so, x.reshape(b * s, d)).reshape(b, s, d)   # attention + x
        hq, sh, _, _ = _cabi.add_rmsnorm_quantize_int8(h, self.post_attention_norm.weight,
                                                       self.post_attention_norm.norm_eps)
        if f.gu_blocked:
            # gate|up in 64-row blocks: a long block forms up * silu(gate) in the GEMM's epilogue
            mq, sm, _ = _cabi.mm_int8_swiglu(hq, f.wgu, sh, f.sgu)
        else:
            gu = _cabi.mm_int8(hq, f.wgu, sh, f.sgu)             # [B*S, gate | up]
            w = f.wgu.size(0) // 2
            mq, sm, _ = _cabi.silu_mul_quantize_int8(gu[:, :w], gu[:, w:])
        return _cabi.mm_int8_resid(mq, f.wdown, sm, f.sdown, h.reshape(b * s, d)).reshape(b, s, d)   # mlp + h


class AutoRegressiveLM(nn.Module):
    def __init__(self, config: AutoRegressiveLMConfig):
        super().__init__()
        self.config = config
        rope_dim = config.hidden_size // config.num_attention_heads
        self.register_buffer(
            "freqs_cis", get_rotary_emb(rope_dim, config.max_position_embeddings,
                                        rotary_base(config.rope_theta, rope_dim, getattr(config, "rope_scaling", None))),
            persistent=False)
        self.embed_tokens = Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList(
            [DecoderBlock(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps)
        self.lm_head = Linear(config.hidden_size, config.vocab_size)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.embed_tokens.weight
        self.apply(lambda m: m.reset_parameters() if hasattr(m, "reset_parameters") else None)
        self.fused_int8 = None  # set by fuse_int8_weights

    def forward(self, input_ids: Tensor, kv_cache: Optional[DenseKVCache] = None,
                positions: Optional[Tensor] = None) -> Dict[str, Tensor]:
        """``input_ids [batch, seq]``. Without a cache: causal forward over the block.
        With a cache: the block's tokens sit at ``positions`` (``[seq]`` int64, on the
        device), keys/values are written there and every query attends to cache
        entries at positions <= its own."""
        if input_ids.ndim != 2:
            raise ValueError("input_ids must be [batch, seq_len]")
        b, s = input_ids.shape
        x = self.embed_tokens(input_ids)
        if positions is None:
            positions = torch.arange(s, device=input_ids.device)
        rotary = self.freqs_cis.index_select(0, positions).unsqueeze(0).float()
        key_mask = None
        if kv_cache is not None:
            key_mask = _KeyMask(positions, kv_cache.max_len,
                                self.config.num_attention_heads // self.config.num_key_value_heads)
        if self.fused_int8 is not None and _fused_int8_active(x):
            from astrai_amd.extension import _cabi
            for layer in self.layers:
                x = layer._forward_fused_int8(x, rotary, kv_cache, positions, key_mask)
            hq, sh, _, hidden = _cabi.add_rmsnorm_quantize_int8(x, self.norm.weight, self.norm.norm_eps,
                                                                None, True)
            logits = _cabi.mm_int8(hq, self.fused_int8.wlm, sh, self.fused_int8.slm).reshape(b, s, -1)
            return {"logits": logits, "hidden_states": hidden}
        for layer in self.layers:
            x = layer(x, rotary, kv_cache, positions, key_mask)
        hidden = self.norm(x)
        return {"logits": self.lm_head(hidden), "hidden_states": hidden}


def _fused_int8_active(x: Tensor) -> bool:
    from astrai_amd.extension import w8a8
    return w8a8.int8_linear_enabled() and x.is_cuda and x.dtype == torch.bfloat16


@torch.no_grad()
def fuse_int8_weights(model: AutoRegressiveLM) -> int:
    """Quantize every projection per output channel (through the int8 policy's weight
    cache, as ``w8a8.prepare_int8_weights`` does) and store q|k|v and gate|up as one
    int8 matrix each on the block. While ``w8a8.int8_autocast`` is on, blocks then take
    the fused path. Returns the number of int8 matrices held. Call again after
    changing weights."""
    from astrai_amd.extension import _cabi, w8a8

    cfg = model.config
    for what, width in (("hidden_size", cfg.hidden_size), ("intermediate_size", cfg.intermediate_size)):
        if not _cabi.fused_rows_supported(width):
            raise ValueError(f"fuse_int8_weights: {what} {width} is outside what the fused producers take "
                             f"(a multiple of 8, at most {_cabi.FUSED_ROW_MAX}); use the Linear-by-Linear "
                             "int8 path (w8a8.prepare_int8_weights) for this model")
    state = w8a8.int8_state()

    def cat(*linears):
        # the policy cache quantizes on first use and returns what it holds otherwise
        # (e.g. the integers an int8 checkpoint installed)
        parts = [state.get_weight(l.weight) for l in linears]
        return torch.cat([p[0] for p in parts]).contiguous(), torch.cat([p[1] for p in parts]).contiguous()

    n = 0
    for blk in model.layers:
        att, mlp = blk.attention, blk.mlp
        wqkv, sqkv = cat(att.q_proj, att.k_proj, att.v_proj)
        wo, so = cat(att.o_proj)
        gu_blocked = cfg.intermediate_size % _cabi.SWIGLU_BLOCK == 0
        if gu_blocked:
            (wg, sg), (wu, su) = state.get_weight(mlp.gate.weight), state.get_weight(mlp.up.weight)
            wgu, sgu = _cabi.swiglu_block_rows(wg, wu), _cabi.swiglu_block_rows(sg, su)
        else:
            wgu, sgu = cat(mlp.gate, mlp.up)
        wdown, sdown = cat(mlp.down)
        blk.fused_int8 = SimpleNamespace(wqkv=wqkv, sqkv=sqkv, wo=wo, so=so, wgu=wgu, sgu=sgu,
                                         gu_blocked=gu_blocked, wdown=wdown, sdown=sdown)
        n += 4
    wlm, slm = cat(model.lm_head)
    model.fused_int8 = SimpleNamespace(wlm=wlm, slm=slm)
    return n + 1


def unfuse_int8_weights(model: AutoRegressiveLM) -> None:
    for blk in model.layers:
        blk.fused_int8 = None
    model.fused_int8 = None


@torch.no_grad()
def greedy_generate(model: AutoRegressiveLM, prompt_ids: Tensor, steps: int,
                    use_graph: bool = False, warmup_steps: int = 2) -> Tensor:
    """Prefill ``prompt_ids [batch, prompt_len]`` then ``steps`` greedy (argmax) decode
    steps; returns the generated ids ``[batch, steps]``. With ``use_graph`` the decode
    step is captured after ``warmup_steps`` eager steps and replayed
    (the reference's warm -> capture -> replay pattern, inference/runtime/graph.py:86-100)."""
    b, p = prompt_ids.shape
    dev = prompt_ids.device
    dtype = model.embed_tokens.weight.dtype
    cache = DenseKVCache(model.config, b, p + steps, dev, dtype)
    logits = model(prompt_ids, cache, torch.arange(p, device=dev))["logits"]
    tok = logits[:, -1].argmax(-1)
    out = torch.empty(b, steps, dtype=torch.long, device=dev)
    cur = tok.clone().reshape(b, 1)
    pos = torch.full((1,), p, dtype=torch.long, device=dev)

    def step():
        lg = model(cur, cache, pos)["logits"]
        return lg[:, -1].argmax(-1)

    graph = None
    nxt_static = None
    for i in range(steps):
        out[:, i] = cur[:, 0]
        if i + 1 == steps:
            break
        if use_graph and graph is None and i >= warmup_steps:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                nxt_static = step()
            graph.replay()  # capture records the step without running it
            nxt = nxt_static
        elif graph is not None:
            graph.replay()
            nxt = nxt_static
        else:
            nxt = step()
        cur.copy_(nxt.reshape(b, 1))
        pos.add_(1)
    return out
