"""Pins the decoder oracle with what the mathematics fixes, on CPU."""

import torch

from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig, DenseKVCache
from oracle import decoder_oracle as D

CFG = AutoRegressiveLMConfig(vocab_size=97, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                             num_key_value_heads=2, intermediate_size=96, max_position_embeddings=32)


def test_rotary_is_a_rotation_with_relative_position_property():
    torch.manual_seed(0)
    fc = D.rotary_table(16, 32, 10000.0)
    q = torch.randn(1, 32, 1, 16)
    k = torch.randn(1, 32, 1, 16)
    # same vector placed at every position
    q[:] = q[:, :1]
    k[:] = k[:, :1]
    rq, rk = D.apply_rotary(q, fc[None]), D.apply_rotary(k, fc[None])
    torch.testing.assert_close(rq.norm(dim=-1), q.norm(dim=-1), rtol=1e-5, atol=1e-5)  # norm preserved
    torch.testing.assert_close(rq[:, 0], q[:, 0])                                       # position 0 = identity
    # <R_m q, R_n k> depends on m - n only
    d1 = (rq[0, 5, 0] * rk[0, 2, 0]).sum()
    d2 = (rq[0, 20, 0] * rk[0, 17, 0]).sum()
    torch.testing.assert_close(d1, d2, rtol=1e-4, atol=1e-4)
    # adjacent pairs rotate by angle pos * base^(-2i/dim): check pair 0 at position 1 (angle 1 rad)
    x = torch.zeros(1, 2, 1, 16)
    x[0, 1, 0, 0] = 1.0
    y = D.apply_rotary(x, fc[None, :2])
    torch.testing.assert_close(y[0, 1, 0, :2], torch.tensor([torch.cos(torch.tensor(1.0)), torch.sin(torch.tensor(1.0))]))


def test_repeat_kv_repeats_each_head_in_place():
    x = torch.arange(2 * 3).float().reshape(1, 1, 2, 3)
    y = D.repeat_kv(x, 2)
    assert y.shape == (1, 1, 4, 3)
    assert torch.equal(y[0, 0, 0], y[0, 0, 1]) and torch.equal(y[0, 0, 2], y[0, 0, 3])
    assert torch.equal(y[0, 0, 0], x[0, 0, 0]) and torch.equal(y[0, 0, 2], x[0, 0, 1])


def test_oracle_bf16_path_equals_the_modules_on_cpu():
    """With stock bf16 linears the functional oracle and the nn.Module decoder are the
    same computation written twice (complex vs real rotary, different head plumbing)."""
    torch.manual_seed(1)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, CFG.vocab_size, (2, 9))
    with torch.no_grad():
        want = D.forward(sd, CFG, ids, D.bf16_linear_fn(sd))
        got = model(ids)["logits"]
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)


def test_causality_and_prefill_decode_contract():
    torch.manual_seed(2)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    lin = D.int8_linear_fn(sd)
    ids = torch.randint(0, CFG.vocab_size, (1, 8))
    full = D.forward(sd, CFG, ids, lin)
    # causal: logits at position t do not depend on later tokens
    ids2 = ids.clone()
    ids2[0, 6:] = (ids2[0, 6:] + 1) % CFG.vocab_size
    part = D.forward(sd, CFG, ids2, lin)
    assert torch.equal(full[:, :6], part[:, :6])
    assert not torch.equal(full[:, 6:], part[:, 6:])
    # the module's prefill-then-decode equals its own full forward (dense cache contract,
    # the analogue of tests/module/test_model_forward.py:71-115 in the reference)
    with torch.no_grad():
        whole = model(ids)["logits"]
        cache = DenseKVCache(CFG, 1, 8, "cpu", torch.bfloat16)
        pre = model(ids[:, :5], cache, torch.arange(5))["logits"]
        dec = [model(ids[:, t:t + 1], cache, torch.tensor([t]))["logits"] for t in range(5, 8)]
    torch.testing.assert_close(torch.cat([pre] + dec, 1).float(), whole.float(), atol=2e-2, rtol=2e-2)


def test_int8_path_tracks_bf16_path():
    torch.manual_seed(3)
    model = AutoRegressiveLM(CFG).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    ids = torch.randint(0, CFG.vocab_size, (2, 12))
    a = D.forward(sd, CFG, ids, D.int8_linear_fn(sd)).float().flatten()
    b = D.forward(sd, CFG, ids, D.bf16_linear_fn(sd)).float().flatten()
    assert torch.nn.functional.cosine_similarity(a, b, dim=0).item() > 0.99
