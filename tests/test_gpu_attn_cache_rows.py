"""The general paged kernel addressed over the dense head-major KV cache (one KV head of one
sequence = one sequence of a one-head pool), for the head shapes the tuned dense kernels do
not take, against the oracle's float32 attention."""

import pytest
import torch

from oracle import decoder_oracle as D
from tests.test_gpu_attn_prefill import _close

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("b,h,hkv,d,s,max_len,start", [
    (3, 4, 2, 64, 1, 40, 17),      # decode, grouping 2
    (2, 8, 1, 64, 1, 300, 299),    # decode, grouping 8, cache exactly full
    (2, 6, 6, 32, 1, 70, 0),       # decode, no grouping, first token
    (1, 16, 1, 256, 1, 130, 77),   # decode, grouping 16, head_dim 256
    (3, 4, 2, 64, 17, 64, 0),      # prefill from an empty cache
    (2, 8, 2, 64, 70, 200, 100),   # chunked prefill: two row tiles, keys before the block
    (2, 3, 1, 32, 5, 40, 11),      # grouping 3
    (1, 4, 2, 256, 33, 64, 9),
    (2, 4, 4, 128, 12, 50, 3),     # head_dim 128 without grouping (not a tuned shape)
])
def test_attn_cache_rows_against_oracle(b, h, hkv, d, s, max_len, start):
    from astrai_amd.extension import _cabi
    print(f"case b={b} h={h}/{hkv} d={d} s={s} max_len={max_len} start={start}", flush=True)
    g = torch.Generator().manual_seed(b * 1000 + h * 100 + d + s)
    q = torch.randn(b, h, s, d, generator=g).to(torch.bfloat16)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    pos = torch.arange(start, start + s, dtype=torch.long)
    last = start + s - 1
    kc[:, :, last + 1:] = float("nan")   # what lies behind the newest position is never read
    vc[:, :, last + 1:] = float("nan")
    got = _cabi.attn_cache_rows(q.to(DEV), kc.to(DEV), vc.to(DEV), pos.to(DEV))
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[:, :, last + 1:] = 0
    vc2[:, :, last + 1:] = 0
    want = D.attn_cached(q, kc2, vc2, pos)
    assert got.shape == (b, s, h * d) and got.dtype == torch.bfloat16
    _close(got, want, "cache rows")


def test_attn_cache_rows_position_past_the_cache_reads_the_cache_and_nothing_else():
    """A model that runs past its cache hands over positions >= max_len (the cache-write kernels
    skip those): the context is clamped to the cache, so the newest token then sees exactly the
    max_len cached keys -- the output of position max_len - 1 -- and no key of the neighbouring
    (sequence, KV head) pair, which directly follows in memory."""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(5)
    b, h, hkv, d, max_len = 3, 4, 2, 64, 48
    q = torch.randn(b, h, 1, d, generator=g).to(torch.bfloat16).to(DEV)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16).to(DEV)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16).to(DEV)
    at_end = _cabi.attn_cache_rows(q, kc, vc, torch.tensor([max_len - 1], device=DEV))
    for past in (max_len, max_len + 5, 10 * max_len):
        got = _cabi.attn_cache_rows(q, kc, vc, torch.tensor([past], device=DEV))
        assert torch.equal(got, at_end), past
    _close(at_end, D.attn_cached(q.cpu(), kc.cpu(), vc.cpu(), torch.tensor([max_len - 1])), "full cache")


def test_attn_cache_rows_scattered_positions():
    """Positions need not be consecutive: every row sees the keys at positions <= its own."""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(77)
    b, h, hkv, d, max_len = 2, 4, 2, 64, 96
    pos = torch.tensor([3, 10, 11, 40, 41, 80], dtype=torch.long)
    q = torch.randn(b, h, len(pos), d, generator=g).to(torch.bfloat16)
    kc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    vc = torch.randn(b, hkv, max_len, d, generator=g).to(torch.bfloat16)
    got = _cabi.attn_cache_rows(q.to(DEV), kc.to(DEV), vc.to(DEV), pos.to(DEV))
    _close(got, D.attn_cached(q, kc, vc, pos), "scattered positions")


def test_head_dim_64_decoder_runs_the_general_kernel(monkeypatch):
    """A fused head_dim-64 decoder with a cache runs attn_cache_rows (prefill block and decode
    steps, graph replay included), never stock SDPA, and stays on the oracle."""
    from astrai_amd.extension import _cabi, w8a8
    from astrai_amd.model import DenseKVCache, fuse_int8_weights, greedy_generate
    from tests.test_gpu_decoder import _Spy, _model
    cfg, model = _model(21, vocab_size=512, hidden_size=256, num_hidden_layers=2, num_attention_heads=4,
                        num_key_value_heads=2, intermediate_size=512, max_position_embeddings=64)
    sd = {k: v.detach().clone() for k, v in model.state_dict().items()}
    ids = torch.randint(0, cfg.vocab_size, (3, 20), generator=torch.Generator().manual_seed(21))
    want = D.forward(sd, cfg, ids, D.int8_linear_fn(sd)).float()
    gm, gids = model.to(DEV), ids.to(DEV)
    w8a8.int8_state().reset()
    spy = _Spy(monkeypatch, ("attn_cache_rows", "attn_decode", "attn_prefill"))
    with torch.no_grad(), w8a8.int8_autocast(True):
        fuse_int8_weights(gm)
        spy.take()
        cache = DenseKVCache(cfg, 3, 20, DEV, torch.bfloat16)
        pre = gm(gids[:, :13], cache, torch.arange(13, device=DEV))["logits"]
        dec = [gm(gids[:, t:t + 1], cache, torch.tensor([t], device=DEV))["logits"] for t in range(13, 20)]
        c = spy.take()
        assert c["attn_cache_rows"] == 2 * 8 and c["sdpa"] == 0 and c["attn_decode"] == 0 and c["attn_prefill"] == 0, c
        eager = greedy_generate(gm, gids[:, :9], 8, use_graph=False)
        graph = greedy_generate(gm, gids[:, :9], 8, use_graph=True)
        assert spy.take()["sdpa"] == 0
    w8a8.int8_state().reset()
    got = torch.cat([pre] + dec, 1).float().cpu()
    cos = torch.nn.functional.cosine_similarity(got.flatten(), want.flatten(), dim=0).item()
    assert cos > 0.999, cos
    assert (got - want).abs().max().item() <= 0.05 * want.abs().max().item()
    assert torch.equal(eager, graph)
