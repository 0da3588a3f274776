"""Host logic that needs no GPU: registry, scaling recipes, autocast context,
per-tensor meta, op-level argument errors -- the CPU-verifiable half of the
reference's tests/extension/test_fp8_mma.py:206-259, against this backend."""

import pytest
import torch

import astrai_amd.extension as ext
from astrai_amd.extension import w8a8
from astrai_amd.extension.fp8 import (
    DelayedScaling,
    DynamicScaling,
    FP8Format,
    FP8TensorMeta,
    fp8_autocast,
    fp8_state,
)
from astrai_amd.extension.ops import fp8 as ops_fp8
from astrai_amd.extension.ops import fp8_block as ops_blk
from astrai_amd.extension.ops import int8 as ops_int8


def test_registry_names_and_modules():
    assert "fp8_mm" in ext.KERNEL_NAMES and "int8_mm" in ext.KERNEL_NAMES
    assert ext.is_available("fp8_mm")
    assert not ext.is_available("no_such_kernel") and ext.get_module("no_such_kernel") is None
    mod = ext.get_module("fp8_mm")
    for name in ("fp8_mm", "quantize_bf16", "mm_fp8", "linear_forward_fp8", "linear_backward_fp8"):
        assert callable(getattr(mod, name))  # csrc/kernels/fp8/mm.cu:350-369


def test_recipe_scale_from_history(golden):
    for r in golden("reference_kats.json")["recipe"]:
        hist = torch.tensor(r["hist"])
        rec = (DelayedScaling(history_len=len(r["hist"]), margin=r["margin"])
               if len(r["hist"]) > 1 else DynamicScaling())
        assert torch.allclose(rec.scale_from_history(hist, r["fmt"]), torch.tensor(r["scale"]))


def test_fp8_format_enum():
    assert FP8Format.HYBRID.fwd() == "e4m3" and FP8Format.HYBRID.bwd() == "e5m2"
    assert FP8Format.E4M3.fwd() == FP8Format.E4M3.bwd() == "e4m3"
    assert FP8Format.E5M2.fwd() == FP8Format.E5M2.bwd() == "e5m2"


def test_fp8_autocast_context_nests_and_restores():
    state = fp8_state()
    prev = (state.enabled, state.recipe, state.fp8_format)
    try:
        with fp8_autocast(enabled=True, fp8_format="hybrid", update_interval=8):
            assert state.enabled
            assert isinstance(state.recipe, DelayedScaling) and state.recipe.history_len == 8
            assert state.fp8_format is FP8Format.HYBRID
            with fp8_autocast(enabled=True, recipe=DynamicScaling(), fp8_format="e4m3"):
                assert isinstance(state.recipe, DynamicScaling)
                assert state.fp8_format is FP8Format.E4M3
            assert state.fp8_format is FP8Format.HYBRID
        assert not state.enabled
    finally:
        state.enabled, state.recipe, state.fp8_format = prev


def test_fp8_tensor_meta_delayed_update(golden):
    kat = golden("reference_kats.json")["meta_update"]
    meta = FP8TensorMeta(torch.device("cpu"), DelayedScaling(history_len=4, margin=0))
    w = torch.randn(8, 8)
    meta.init_w(w, "e4m3")
    assert meta.w_init and not meta.x_init
    torch.testing.assert_close(meta.w_scale, (w.abs().amax() / 448.0).reshape(1))
    meta.update_w(torch.tensor([kat["amax"]]), "e4m3")
    torch.testing.assert_close(meta.w_scale, torch.tensor(kat["scale"]).reshape(1))
    assert meta.w_idx == 1 and meta.w_hist[0].item() == kat["amax"]


def test_ring_wraps_and_forgets_old_peaks():
    meta = FP8TensorMeta(torch.device("cpu"), DelayedScaling(history_len=2))
    meta.init_x(torch.tensor([1.0]), "e4m3")
    for a in (8.0, 2.0, 1.0):
        meta.update_x(torch.tensor([a]), "e4m3")
    # window now holds (1.0, 2.0): the 8.0 peak has rotated out
    torch.testing.assert_close(meta.x_scale, torch.tensor([2.0 / 448.0]))


def test_reference_ops_cpu_kernels(golden):
    """The reference registers cpu kernels on its two dispatcher ops and tests them
    with these vectors (tests/extension/test_fp8_mma.py:262-293)."""
    kats = golden("reference_kats.json")
    torch.manual_seed(0)
    x = torch.randn(16, 32, dtype=torch.bfloat16)
    x8, amax = ops_fp8.quantize_bf16(x, torch.tensor([kats["quantize_scale"]]), "e4m3")
    assert x8.dtype == torch.float8_e4m3fn
    # dividing by 0.5 is an exact doubling, so the expected codes are the cast of 2x
    assert torch.equal(x8.view(torch.uint8), (x.float() * 2).to(torch.float8_e4m3fn).view(torch.uint8))
    torch.testing.assert_close(amax, x.abs().amax().float().reshape(1))
    x5, _ = ops_fp8.quantize_bf16(x, torch.tensor([1.0]), "e5m2")
    assert x5.dtype == torch.float8_e5m2
    k = kats["mm_fp8_cpu"]
    a8 = torch.tensor(k["a8"]).to(torch.float8_e4m3fn)
    b8 = torch.tensor(k["b8"]).to(torch.float8_e4m3fn)
    out = ops_fp8.mm_fp8(a8, b8, torch.tensor([k["sa"]]), torch.tensor([k["sb"]]))
    assert out.dtype == torch.bfloat16 and out.tolist() == k["out_bf16"]
    k = kats["mm_fp8_fp8_out_cpu"]
    out8 = ops_fp8.mm_fp8(a8, b8, torch.tensor([k["sa"]]), torch.tensor([k["sb"]]),
                          out_dtype="e4m3", out_scale=torch.tensor([k["out_scale"]]))
    assert out8.dtype == torch.float8_e4m3fn and out8.float().tolist() == k["out_e4m3"]
    # an all-zero input: the floor keeps the amax positive (ops/fp8.py:81)
    _, amax0 = ops_fp8.quantize_bf16(torch.zeros(2, 2, dtype=torch.bfloat16), torch.tensor([1.0]))
    assert float(amax0) == pytest.approx(1e-12)


def test_added_ops_have_no_cpu_arithmetic():
    x = torch.randn(4, 8).to(torch.bfloat16)
    a8 = torch.zeros(2, 2, dtype=torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="no CPU"):
        ops_int8.quantize_int8_per_token(x)
    with pytest.raises(RuntimeError, match="no CPU"):
        ops_blk.mm_fp8_blockscaled(a8, a8, torch.ones(2, 1), torch.ones(1, 1))


def test_argument_errors_match_the_reference_types():
    x = torch.randn(2, 2).to(torch.bfloat16)
    with pytest.raises(ValueError, match="fmt must be one of"):
        ops_fp8.quantize_bf16(x, torch.tensor([1.0]), "e3m4")   # ops/fp8.py:44-48
    a8 = torch.zeros(2, 2, dtype=torch.float8_e4m3fn)
    with pytest.raises(ValueError, match="out_dtype must be one of"):
        ops_fp8.mm_fp8(a8, a8, torch.ones(1), torch.ones(1), out_dtype="fp16")  # :150-153
    with pytest.raises(TypeError, match="bf16 tensors only"):
        ops_fp8.linear_forward_fp8(x.float(), x, None, torch.ones(1), torch.ones(1))  # :162-163


def test_fake_kernels_give_shapes_for_tracing():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x = torch.empty(6, 32, dtype=torch.bfloat16)
        x8, amax = torch.ops.custom.fp8_quantize(x, torch.empty(1), 1)
        assert x8.dtype == torch.float8_e5m2 and x8.shape == (6, 32) and amax.shape == (1,)
        a = torch.empty(6, 32, dtype=torch.float8_e4m3fn)
        b = torch.empty(10, 32, dtype=torch.float8_e4m3fn)
        assert torch.ops.custom.fp8_gemm(a, b, torch.empty(1), torch.empty(1)).shape == (6, 10)
        assert torch.ops.custom.fp8_gemm(a, b, torch.empty(1), torch.empty(1), 1, torch.empty(1)).dtype == torch.float8_e4m3fn
        xq, s = torch.ops.custom.int8_quantize_per_token(torch.empty(2, 3, 32, dtype=torch.bfloat16))
        assert xq.shape == (6, 32) and s.shape == (6, 1)
        ai = torch.empty(6, 32, dtype=torch.int8)
        bi = torch.empty(10, 32, dtype=torch.int8)
        out = torch.ops.custom.int8_gemm(ai, bi, torch.empty(6, 1), torch.empty(10))
        assert out.shape == (6, 10) and out.dtype == torch.bfloat16


def test_linear_override_leaves_cpu_and_disabled_calls_alone():
    x, w = torch.randn(3, 8), torch.randn(5, 8)
    with fp8_autocast(enabled=True), w8a8.int8_autocast(True):
        y = torch.nn.functional.linear(x, w)     # CPU tensors never reach the CUDA-key hook
    torch.testing.assert_close(y, x @ w.t())
    assert not w8a8.int8_linear_enabled() and not fp8_state().enabled


def test_int8_autocast_restores():
    assert not w8a8.int8_linear_enabled()
    with w8a8.int8_autocast(True):
        assert w8a8.int8_linear_enabled()
        with w8a8.int8_autocast(False):
            assert not w8a8.int8_linear_enabled()
        assert w8a8.int8_linear_enabled()
    assert not w8a8.int8_linear_enabled()


def test_fp8_scaling_state_survives_a_checkpoint(tmp_path):
    """Delayed scaling resumed from ``save_fp8_scaling`` continues exactly where the saved run
    stood: same histories, cursors, steps, and the same steps after further updates as a run
    that was never interrupted."""
    import json
    from astrai_amd.model.checkpoint import load_fp8_scaling, save_fp8_scaling

    def feed(model, amaxes):
        st = fp8_state()
        for p, vals in zip(model.parameters(), amaxes):
            meta = st.get_weight_meta(p)
            if not meta.w_init:
                meta.init_w(p, "e4m3")
            for a in vals:
                meta.update_x(torch.tensor([a]), "e4m3")
                meta.update_g(torch.tensor([a * 0.01]), "e5m2")
                meta.update_w(torch.tensor([a * 0.5]), "e4m3")

    def snapshot(model):
        st = fp8_state()
        out = []
        for p in model.parameters():
            m = st.peek_weight_meta(p)
            out.append(None if m is None else
                       [t.clone() for t in (m.w_hist, m.x_hist, m.g_hist, m.w_scale, m.x_scale, m.g_scale)]
                       + [m.w_idx, m.x_idx, m.g_idx, m.w_init])
        return out

    def same(a, b):
        return all((x is None and y is None) or all(torch.equal(u, v) if torch.is_tensor(u) else u == v
                                                    for u, v in zip(x, y)) for x, y in zip(a, b))

    torch.manual_seed(0)
    model = torch.nn.Sequential(torch.nn.Linear(8, 4, bias=False), torch.nn.Linear(4, 2, bias=False))
    first = [[3.0, 7.0, 2.0, 9.0, 1.0], [0.5, 0.25]]
    later = [[4.0, 4.0, 30.0], [0.125, 2.0, 1.0, 1.0, 1.0]]
    st = fp8_state()
    st.reset()
    try:
        with fp8_autocast(update_interval=4, margin=1):
            feed(model, first)
            before = snapshot(model)
            assert save_fp8_scaling(model, str(tmp_path)) == 2
            feed(model, later)
            uninterrupted = snapshot(model)
            # a fresh process: no state; the weights are the same tensors of a re-built model
            st._metas.clear()
            assert all(s is None for s in snapshot(model))
            assert load_fp8_scaling(model, str(tmp_path)) == 2
            assert same(snapshot(model), before)
            feed(model, later)
            assert same(snapshot(model), uninterrupted)
        info = json.loads((tmp_path / "meta.json").read_text())["fp8_scaling"]
        assert info == {"recipe": "DelayedScaling", "history_len": 4, "margin": 1, "fp8_format": "hybrid",
                        "parameters": 2}
        with fp8_autocast(update_interval=8):
            with pytest.raises(ValueError, match="slots"):
                load_fp8_scaling(model, str(tmp_path))
    finally:
        st.reset()


def test_int8_weight_cache_is_tied_to_the_tensor_object(monkeypatch):
    """A cached int8 form belongs to one tensor object at one version: another
    tensor with the same address, shape and dtype (a freed weight's memory
    reused) must be quantized afresh, an in-place update too."""
    calls = []

    def fake_quantize(w):
        calls.append(w)
        return (torch.full(w.shape, len(calls), dtype=torch.int8),
                torch.full((w.size(0),), float(len(calls))))

    monkeypatch.setattr(w8a8, "quantize_int8_per_channel", fake_quantize)
    st = w8a8.Int8State()
    w1 = torch.zeros(4, 8, dtype=torch.bfloat16)
    q1, _ = st.get_weight(w1)
    assert st.get_weight(w1)[0] is q1 and len(calls) == 1          # hit
    alias = w1.detach()                                            # same address, shape, dtype, version
    assert alias.data_ptr() == w1.data_ptr() and alias is not w1
    assert st.lookup(alias) is None
    q2, s2 = st.get_weight(alias)
    assert len(calls) == 2 and int(q2[0, 0]) == 2 and float(s2[0]) == 2.0
    assert st.lookup(w1) is None                                   # the slot now belongs to `alias`
    alias.add_(1)                                                  # version bump
    assert st.lookup(alias) is None
    st.get_weight(alias)
    assert len(calls) == 3
    # an installed form (checkpoint load) obeys the same identity rule
    w3 = torch.zeros(2, 8, dtype=torch.bfloat16)
    st.put_weight(w3, torch.ones(2, 8, dtype=torch.int8), torch.ones(2))
    assert st.lookup(w3) is not None and st.lookup(w3.detach()) is None
    # entries of dead tensors are dropped on the next store
    del w3
    st.put_weight(w1, torch.ones(4, 8, dtype=torch.int8), torch.ones(4))
    assert all(e[0]() is not None for e in st._weights.values())


def test_cache_context_len_is_clamped_to_the_cache():
    """attn_cache_rows never addresses more keys than the cache holds, whatever the positions say."""
    from astrai_amd.extension._cabi import cache_context_len
    for pos, max_len, want in (([0], 8, 1), ([3, 4, 5], 8, 6), ([7], 8, 8), ([8], 8, 8), ([100, 3], 8, 8), ([2, 9], 16, 10)):
        got = cache_context_len(torch.tensor(pos), max_len)
        assert got.dtype == torch.int32 and got.item() == want, (pos, max_len)


def test_weight_side_padding_is_made_once_and_follows_writes():
    """K % 16 != 0 products pad both operands with zero codes; the weight's padded form is kept while
    that tensor lives unmodified (a Linear's codes are one long-lived tensor), not rebuilt per call."""
    from astrai_amd.extension import _cabi
    a = torch.randint(-5, 5, (200, 1000), dtype=torch.int8)
    w = torch.randint(-5, 5, (300, 1000), dtype=torch.int8)
    a1, w1, k1 = _cabi._pad_k(a, w)
    a2, w2, k2 = _cabi._pad_k(a, w)
    assert k1 == k2 == 1024 and w1 is w2 and a1 is not a2
    assert torch.equal(w1[:, :1000], w) and not w1[:, 1000:].any() and not a1[:, 1000:].any()
    w[0, 0] += 1                                   # a write: the kept form is stale
    _, w3, _ = _cabi._pad_k(a, w)
    assert w3 is not w1 and torch.equal(w3[:, :1000], w)
    n = len(_cabi._padded_weights)
    del w, w1, w2, w3
    _cabi._pad_k(a, torch.zeros(300, 1000, dtype=torch.int8))   # a new weight: dead entries are dropped
    assert len(_cabi._padded_weights) <= n
    small, ws, ks = _cabi._pad_k(a[:2, :40], a[:3, :40])        # too small to repay a copy
    assert ks == 40 and small.shape == (2, 40)
