"""The reference's dense attention entry points (attn_decode / attn_prefill on q, k, v tensors
in either layout, boolean is_causal, optional masks) and its rotary_emb entry, through the
registry and the ops wrappers, against the oracle."""

import pytest
import torch

from oracle import decoder_oracle as D
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _close(got, want, what):
    """Prefill bound (probabilities and output rounded to bf16): |y - ref| <= 2e-2 |ref| + four
    bf16 ulps at rms(ref)."""
    g, w = got.float().cpu(), want.float().cpu()
    assert g.shape == w.shape, (g.shape, w.shape)
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    rms = w.pow(2).mean().sqrt().item()
    err = (g - w).abs()
    bad = err > 2e-2 * w.abs() + 2.0 ** -6 * rms
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance; worst {err.max().item():.4g}"


def _qkv(b, lq, lk, h, hkv, seed, layout=1):
    g = torch.Generator().manual_seed(seed)
    mk = lambda l, n: torch.randn(b, l, n, 128, generator=g).to(torch.bfloat16)
    q, k, v = mk(lq, h), mk(lk, hkv), mk(lk, hkv)
    if layout == 0:
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    return q, k, v


def test_registry_lists_the_reference_kernel_names():
    from astrai_amd.extension import KERNEL_NAMES, get_module, is_available
    for name in ("attn_decode", "attn_prefill", "attn_paged_decode", "attn_paged_prefill", "rotary_emb", "fp8_mm"):
        assert name in KERNEL_NAMES and is_available(name)
        assert callable(getattr(get_module(name), name))      # csrc/CMakeLists.txt:55-62: module name = entry name


@pytest.mark.parametrize("h,hkv", [(16, 4), (8, 8), (16, 2)])
@pytest.mark.parametrize("is_causal", [False, True])
def test_ops_attn_decode_blhd(h, hkv, is_causal):
    from astrai_amd.extension import ops
    q, k, v = _qkv(3, 1, 77, h, hkv, seed=h + hkv)
    got = ops.attn_decode(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=is_causal)
    assert got.shape == q.shape and got.dtype == torch.bfloat16
    assert_bf16_close(got, D.attn_dense(q, k, v), what=f"decode {h}/{hkv}")   # one row: causal sees every key
    g = torch.Generator().manual_seed(3)
    mask = torch.rand(3, 77, generator=g) < 0.6
    mask[2] = False                                      # a hidden sequence: zeros
    for m in (mask, mask[:, None, :]):
        got = ops.attn_decode(q.to(DEV), k.to(DEV), v.to(DEV), mask=m.to(DEV), is_causal=is_causal)
        assert_bf16_close(got, D.attn_dense(q, k, v, mask=m), what=f"decode mask {tuple(m.shape)}")
        assert got[2].abs().sum() == 0


@pytest.mark.parametrize("layout", [0, 1])
def test_registry_attn_decode_layouts_and_offsets(layout):
    """The pybind-level entry: layout code, causal_offset as a key limit (layout_policies.cuh:
    138-141), strided inputs."""
    from astrai_amd.extension import get_module
    fn = get_module("attn_decode").attn_decode
    q, k, v = _qkv(2, 1, 130, 8, 2, seed=11, layout=layout)
    dev = [t.to(DEV) for t in (q, k, v)]
    for off in (-1, 0, 40, 129, 500):
        got = fn(*dev, causal_offset=off, layout=layout)
        assert got.shape == q.shape
        assert_bf16_close(got, D.attn_dense(q, k, v, causal_offset=off, layout=layout), what=f"layout {layout} offset {off}")
    mask = torch.rand(2, 130, generator=torch.Generator().manual_seed(1)) < 0.5
    got = fn(*dev, mask=mask.to(DEV), causal_offset=100, layout=layout)
    assert_bf16_close(got, D.attn_dense(q, k, v, mask=mask, causal_offset=100, layout=layout), what="mask and offset")
    per_head = torch.rand(2, 8, 1, 130, generator=torch.Generator().manual_seed(2)) < 0.5
    got = fn(*dev, mask=per_head.to(DEV), causal_offset=100, layout=layout)
    assert_bf16_close(got, D.attn_dense(q, k, v, mask=per_head, causal_offset=100, layout=layout), what="mask per head")
    # a key tensor that is a window of a longer buffer (non-contiguous)
    g = torch.Generator().manual_seed(5)
    shape = (2, 200, 2, 128) if layout == 1 else (2, 2, 200, 128)
    big_k = torch.randn(shape, generator=g).to(torch.bfloat16)
    big_v = torch.randn(shape, generator=g).to(torch.bfloat16)
    win = (slice(None), slice(20, 150)) if layout == 1 else (slice(None), slice(None), slice(20, 150))
    got = fn(dev[0], big_k.to(DEV)[win], big_v.to(DEV)[win], layout=layout)
    assert_bf16_close(got, D.attn_dense(q, big_k[win], big_v[win], layout=layout), what="window")


@pytest.mark.parametrize("h,hkv,lq,lk", [(8, 2, 70, 70), (16, 4, 33, 150), (4, 2, 128, 128), (16, 2, 5, 64)])
@pytest.mark.parametrize("is_causal", [False, True])
def test_ops_attn_prefill_blhd(h, hkv, lq, lk, is_causal):
    from astrai_amd.extension import ops
    q, k, v = _qkv(2, lq, lk, h, hkv, seed=lq + lk)
    off = lk - lq if is_causal else -1
    got = ops.attn_prefill(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=is_causal)
    assert got.shape == q.shape and got.dtype == torch.bfloat16
    _close(got, D.attn_dense(q, k, v, causal_offset=off), f"prefill {h}/{hkv} {lq}x{lk} causal={is_causal}")
    g = torch.Generator().manual_seed(9)
    m2 = torch.rand(2, lk, generator=g) < 0.7
    m3 = torch.rand(2, lq, lk, generator=g) < 0.7
    m3[1, lq // 2] = False                                # a hidden row: zeros
    for m in (m2, m3):
        got = ops.attn_prefill(q.to(DEV), k.to(DEV), v.to(DEV), mask=m.to(DEV), is_causal=is_causal)
        _close(got, D.attn_dense(q, k, v, mask=m, causal_offset=off), f"prefill mask {tuple(m.shape)}")
    assert got[1, lq // 2].abs().sum() == 0


@pytest.mark.parametrize("layout", [0, 1])
def test_registry_attn_prefill_layouts_offsets_and_4d_masks(layout):
    from astrai_amd.extension import get_module
    fn = get_module("attn_prefill").attn_prefill
    b, lq, lk, h, hkv = 2, 90, 140, 8, 2
    q, k, v = _qkv(b, lq, lk, h, hkv, seed=21, layout=layout)
    dev = [t.to(DEV) for t in (q, k, v)]
    for off in (-1, lk - lq, 0, 10, 1000):               # aligned to the end, to the start, in between, past everything
        got = fn(*dev, causal_offset=off, layout=layout)
        assert got.shape == q.shape
        _close(got, D.attn_dense(q, k, v, causal_offset=off, layout=layout), f"layout {layout} offset {off}")
    g = torch.Generator().manual_seed(2)
    for shape in ((b, 1, 1, lk), (b, h, 1, lk), (b, 1, lq, lk), (b, h, lq, lk)):
        m = torch.rand(shape, generator=g) < 0.6
        got = fn(*dev, mask=m.to(DEV), causal_offset=lk - lq, layout=layout)
        _close(got, D.attn_dense(q, k, v, mask=m, causal_offset=lk - lq, layout=layout), f"4D mask {shape}")
        got = fn(*dev, mask=m.to(DEV), causal_offset=7, layout=layout)
        _close(got, D.attn_dense(q, k, v, mask=m, causal_offset=7, layout=layout), f"4D mask {shape}, offset 7")


def test_dense_entries_reject_what_the_reference_rejects():
    from astrai_amd.extension import get_module
    dec, pre = get_module("attn_decode").attn_decode, get_module("attn_prefill").attn_prefill
    q, k, v = (t.to(DEV) for t in _qkv(2, 1, 16, 8, 2, seed=1))
    with pytest.raises(RuntimeError, match="seq_len must be 1"):
        dec(k[:, :2].repeat(1, 1, 4, 1), k, v, layout=1)
    with pytest.raises(RuntimeError, match="identical shapes"):
        dec(q, k, v[:, :8], layout=1)
    with pytest.raises(RuntimeError, match="4D"):
        dec(q[0], k, v, layout=1)
    with pytest.raises(RuntimeError, match="bf16"):
        dec(q.float(), k, v, layout=1)
    with pytest.raises(RuntimeError, match="divisible"):
        dec(q[:, :, :3], k, v, layout=1)
    with pytest.raises(RuntimeError, match="mask kv_len"):
        dec(q, k, v, mask=torch.ones(2, 15, dtype=torch.bool, device=DEV), layout=1)
    with pytest.raises(RuntimeError, match="mask batch"):
        pre(q, k, v, mask=torch.ones(3, 16, dtype=torch.bool, device=DEV), layout=1)
    with pytest.raises(RuntimeError, match="mask must be bool"):
        pre(q, k, v, mask=torch.ones(2, 16, device=DEV), layout=1)
    with pytest.raises(RuntimeError, match="head_dim"):
        pre(q[..., :48], k[..., :48], v[..., :48], layout=1)


@pytest.mark.parametrize("shape", [(37, 16, 128), (2, 19, 4, 128), (5, 3, 64), (4, 2, 6), (1, 1, 2), (0, 4, 128)])
def test_rotary_emb_equals_the_fp32_tensor_arithmetic(shape):
    """Bit for bit the reference's torch path (astrai/extension/backend/rotary.py:25-33): complex
    multiply in fp32, one rounding to bf16. Packed and dense inputs, head_dim with and without
    16-byte rows, empty input."""
    from astrai_amd.extension import ops
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(shape, generator=g) * 3).to(torch.bfloat16)
    ang = torch.rand(*shape[:-2], shape[-1] // 2, generator=g) * 6.28318
    freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1)
    got = ops.rotary_emb(x.to(DEV), freqs.to(DEV))
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    if x.numel():
        assert torch.equal(got.cpu(), D.apply_rotary(x, freqs))


def test_rotary_emb_large_and_argument_checks():
    from astrai_amd.extension import get_module, ops
    fn = get_module("rotary_emb").rotary_emb
    g = torch.Generator().manual_seed(77)
    x = torch.randn(4, 512, 16, 128, generator=g).to(torch.bfloat16)
    table = D.rotary_table(128, 600, 10000.0)
    pos = torch.randint(0, 600, (4, 512), generator=g)
    freqs = table[pos]                                    # [4, 512, 64, 2]: each token's own row
    got = fn(x.to(DEV), freqs.to(DEV))
    assert torch.equal(got.cpu(), D.apply_rotary(x, freqs))
    # the wrapper copies non-contiguous inputs; the entry refuses them like the reference's
    xt = x.transpose(0, 1)                                # [512, 4, 16, 128] view
    ft = freqs.transpose(0, 1)
    assert torch.equal(ops.rotary_emb(xt.to(DEV), ft.to(DEV)).cpu(), D.apply_rotary(xt, ft))
    xd, fd = x.to(DEV), freqs.to(DEV)
    for args, msg in (((xd.transpose(0, 1), fd), "x must be contiguous"),
                      ((xd, fd.transpose(0, 1)), "freqs_cis must be contiguous"),
                      ((xd.float(), fd), "x must be bf16"), ((xd, fd.double()), "freqs_cis must be f32"),
                      ((xd, fd[0]), "rank"), ((xd, fd[:3]), "mismatch"), ((xd[0, 0], fd[0, 0]), "x must be"),
                      ((xd.cpu(), fd), "CUDA")):
        with pytest.raises(RuntimeError, match=msg):
            fn(*args)


# ---- the general paged kernel: head_dim 32 / 64 / 256, any grouping up to 8 ----

def _paged_case(b, h, hkv, d, kv_lens, q_lens, seed, holes=False):
    g = torch.Generator().manual_seed(seed)
    total_q, pool = sum(q_lens), sum(kv_lens) + 9
    q = torch.randn(total_q, h, d, generator=g).to(torch.bfloat16)
    k_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    v_pool = torch.randn(pool, hkv, d, generator=g).to(torch.bfloat16)
    rows = torch.randperm(b + 2, generator=g)[:b].int()
    table = torch.full((b + 2, max(kv_lens) + 3), -1, dtype=torch.int32)
    perm = torch.randperm(pool, generator=g)
    nxt = 0
    for i in range(b):
        table[rows[i], :kv_lens[i]] = perm[nxt:nxt + kv_lens[i]].int()
        nxt += kv_lens[i]
        if holes and kv_lens[i] > 4:
            table[rows[i], 2] = -1
    k_pool[perm[nxt:]] = float("nan")         # slots no live position maps to must not be read
    v_pool[perm[nxt:]] = float("nan")
    kvp = torch.tensor([0] + torch.tensor(kv_lens).cumsum(0).tolist(), dtype=torch.int32)
    return q, k_pool, v_pool, table, rows, kvp


@pytest.mark.parametrize("d", [32, 64, 256])
@pytest.mark.parametrize("h,hkv", [(2, 1), (4, 4), (6, 2), (8, 1), (16, 4), (16, 1), (24, 2)])
def test_paged_decode_other_head_dims_and_groupings(d, h, hkv):
    """head_dim 64 with 2 heads on 1 KV head is the reference's own test model
    (tests/extension/conftest.py:9-20)."""
    from astrai_amd.extension import ops
    lens = [70, 1, 0, 33, 150]
    args = _paged_case(5, h, hkv, d, lens, [1] * 5, seed=d + h, holes=True)
    dev = [t.to(DEV) for t in args]
    want = D.attn_paged_decode(*args)
    got = ops.attn_paged_decode(*dev, is_causal=True)
    assert got.shape == (5, h, d)
    assert_bf16_close(got, want, what=f"decode d={d} {h}/{hkv}")
    assert got[2].abs().sum() == 0
    mask = torch.rand(5, max(lens) + 3, generator=torch.Generator().manual_seed(d)) < 0.6
    got = ops.attn_paged_decode(*dev, mask=mask.to(DEV), is_causal=True)
    assert_bf16_close(got, D.attn_paged_decode(*args, mask=mask), what=f"decode d={d} {h}/{hkv} mask")
    from astrai_amd.extension import _cabi
    for nsplit in (1, 3):
        got = _cabi.attn_paged_decode(*dev, nsplit=nsplit)
        assert_bf16_close(got, want, what=f"decode d={d} nsplit={nsplit}")


@pytest.mark.parametrize("d,h,hkv", [(64, 2, 1), (64, 4, 4), (32, 8, 1), (256, 4, 2), (128, 4, 4), (128, 6, 2), (64, 16, 2),
                                     (128, 16, 1), (64, 10, 2), (256, 3, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_paged_prefill_other_head_dims_and_groupings(d, h, hkv, causal):
    """The shapes the MFMA prefill kernel does not take (head_dim != 128, or a grouping other
    than 2 / 4 / 8, multi-head attention included) run the general kernel."""
    from astrai_amd.extension import _cabi, ops
    kv_lens, q_lens = [100, 37, 64, 5], [70, 37, 1, 5]
    args = _paged_case(4, h, hkv, d, kv_lens, q_lens, seed=d + h + hkv, holes=True)
    dev = [t.to(DEV) for t in args]
    qo, tb, ti = _cabi.paged_prefill_schedule(q_lens, DEV)
    got = ops.attn_paged_prefill(*dev, qo, tb, ti, is_causal=causal)
    assert got.shape == (sum(q_lens), h, d)
    want = D.attn_paged_prefill(*args, qo.cpu(), causal=causal)
    _close(got, want, f"prefill d={d} {h}/{hkv} causal={causal}")
    off = 0 if causal else -1
    for nsplit in (1, 3):       # 1: workgroups of four row blocks sharing the key tiles; 3: split context + merge
        got = _cabi.attn_paged_prefill(*dev, qo, tb, ti, causal_offset=off, nsplit=nsplit)
        _close(got, want, f"prefill d={d} {h}/{hkv} causal={causal} nsplit={nsplit}")
    g = torch.Generator().manual_seed(d)
    for shape in ((4, max(kv_lens) + 3), (4, 1, max(q_lens), max(kv_lens)), (4, h, max(q_lens), max(kv_lens))):
        mask = torch.rand(shape, generator=g) < 0.6
        want = D.attn_paged_prefill(*args, qo.cpu(), causal=causal, mask=mask)
        for nsplit in (0, 1):
            got = _cabi.attn_paged_prefill(*dev, qo, tb, ti, mask=mask.to(DEV), causal_offset=off, nsplit=nsplit)
            _close(got, want, f"prefill d={d} mask {shape} nsplit={nsplit}")


def test_general_kernel_agrees_with_the_tuned_kernels_where_both_apply():
    """head_dim 128, grouping 4: the rows entry through the C ABI against the tuned paged kernels."""
    import ctypes
    from astrai_amd.extension import _cabi
    lib = _cabi.load()
    kv_lens, q_lens = [300, 64, 129], [300, 1, 60]
    args = _paged_case(3, 16, 4, 128, kv_lens, q_lens, seed=5)
    q, kp, vp, table, rows, kvp = [t.to(DEV) for t in args]
    qo, tb, ti = _cabi.paged_prefill_schedule(q_lens, DEV)
    tuned = _cabi.attn_paged_prefill(q, kp, vp, table, rows, kvp, qo, tb, ti, causal_offset=0)
    out = torch.empty_like(tuned)
    _cabi._paged_rows(lib, q, kp, vp, table, rows, kvp, (qo, tb, ti), (0, 0, 0, 0, 0, 0), out, tb.numel(), 2, True,
                      128 ** -0.5)
    _close(out, tuned, "rows kernel vs MFMA prefill kernel")
    q1 = q[:3].contiguous()
    tuned = _cabi.attn_paged_decode(q1, kp, vp, table, rows, kvp, nsplit=2)
    out = torch.empty_like(tuned)
    _cabi._paged_rows(lib, q1, kp, vp, table, rows, kvp, None, (0, 0, 0, 0, 0, 0), out, 3, 2, False, 128 ** -0.5)
    assert_bf16_close(out, tuned, what="rows kernel vs tuned decode kernel")
    out1 = torch.empty_like(tuned)                 # without a split the waves write the output themselves
    _cabi._paged_rows(lib, q1, kp, vp, table, rows, kvp, None, (0, 0, 0, 0, 0, 0), out1, 3, 1, False, 128 ** -0.5)
    assert_bf16_close(out1, tuned, what="rows kernel, no split")
    outp = torch.empty(q.shape, dtype=q.dtype, device=DEV)
    _cabi._paged_rows(lib, q, kp, vp, table, rows, kvp, (qo, tb, ti), (0, 0, 0, 0, 0, 0), outp, tb.numel(), 1, True,
                      128 ** -0.5)
    _close(outp, _cabi.attn_paged_prefill(q, kp, vp, table, rows, kvp, qo, tb, ti, causal_offset=0), "rows prefill, no split")


@pytest.mark.parametrize("layout", [0, 1])
def test_dense_entries_head_dim_64_like_the_reference_test_model(layout):
    from astrai_amd.extension import get_module
    dec, pre = get_module("attn_decode").attn_decode, get_module("attn_prefill").attn_prefill
    g = torch.Generator().manual_seed(64)
    b, lq, lk, h, hkv, d = 2, 16, 40, 2, 1, 64
    mk = lambda l, n: torch.randn(b, l, n, d, generator=g).to(torch.bfloat16)
    q, k, v = mk(lq, h), mk(lk, hkv), mk(lk, hkv)
    if layout == 0:
        q, k, v = (t.transpose(1, 2).contiguous() for t in (q, k, v))
    dev = [t.to(DEV) for t in (q, k, v)]
    for off in (-1, lk - lq, 0):
        _close(pre(*dev, causal_offset=off, layout=layout), D.attn_dense(q, k, v, causal_offset=off, layout=layout),
               f"prefill layout {layout} offset {off}")
    q1 = q[:, :, :1].contiguous() if layout == 0 else q[:, :1].contiguous()
    got = dec(q1.to(DEV), dev[1], dev[2], causal_offset=lk - 1, layout=layout)
    assert_bf16_close(got, D.attn_dense(q1, k, v, layout=layout), what=f"decode layout {layout}")
    with pytest.raises(RuntimeError, match="head_dim"):
        pre(dev[0][..., :48], dev[1][..., :48], dev[2][..., :48], layout=layout)


@pytest.mark.parametrize("d", [64, 128])
def test_attention_entries_with_nothing_to_do(d):
    """Empty batch, empty schedule, sequences without keys or without query rows: shapes come
    back right, nothing is launched out of bounds, rows without keys are zeros."""
    from astrai_amd.extension import _cabi, get_module, ops
    h, hkv = 4, 2
    kp = torch.randn(16, hkv, d).to(torch.bfloat16).to(DEV)
    table = torch.arange(16, dtype=torch.int32, device=DEV).reshape(2, 8)
    none = torch.zeros(0, dtype=torch.int32, device=DEV)
    zero1 = torch.zeros(1, dtype=torch.int32, device=DEV)
    q0 = torch.zeros(0, h, d, dtype=torch.bfloat16, device=DEV)
    assert ops.attn_paged_decode(q0, kp, kp, table, none, zero1).shape == (0, h, d)
    qo, tb, ti = _cabi.paged_prefill_schedule([], DEV)
    assert ops.attn_paged_prefill(q0, kp, kp, table, none, zero1, qo, tb, ti, is_causal=True).shape == (0, h, d)
    # two sequences: the first has rows but no keys, the second keys but no rows
    q = torch.randn(5, h, d).to(torch.bfloat16).to(DEV)
    rows = torch.arange(2, dtype=torch.int32, device=DEV)
    kvp = torch.tensor([0, 0, 6], dtype=torch.int32, device=DEV)
    qo, tb, ti = _cabi.paged_prefill_schedule([5, 0], DEV)
    for causal in (True, False):
        out = ops.attn_paged_prefill(q, kp, kp, table, rows, kvp, qo, tb, ti, is_causal=causal)
        assert out.shape == (5, h, d) and out.abs().sum() == 0
    out = ops.attn_paged_decode(q[:2].contiguous(), kp, kp, table, rows, kvp)
    assert out[0].abs().sum() == 0 and out[1].abs().sum() > 0
    dec, pre = get_module("attn_decode").attn_decode, get_module("attn_prefill").attn_prefill
    k0 = torch.zeros(2, 0, hkv, d, dtype=torch.bfloat16, device=DEV)
    q4 = torch.randn(2, 3, h, d).to(torch.bfloat16).to(DEV)
    assert pre(q4, k0, k0, layout=1).abs().sum() == 0 and pre(q4, k0, k0, layout=1).shape == q4.shape
    assert dec(q4[:, :1].contiguous(), k0, k0, layout=1).abs().sum() == 0
    assert pre(q4[:0], k0[:0], k0[:0], layout=1).shape == (0, 3, h, d)


def test_general_kernel_random_sweep():
    """Thirty seeded random batches through the general kernel: head_dim, grouping (1..16), ragged
    cached-prefix and new-token counts (some with more rows than keys), causal or not, padding
    slots, every mask form, every split choice; decode on the same pools."""
    from astrai_amd.extension import _cabi
    g = torch.Generator().manual_seed(2718)
    ri = lambda lo, hi: int(torch.randint(lo, hi, (1,), generator=g))
    for i in range(30):
        d = (32, 64, 128, 256)[ri(0, 4)]
        n_rep = (1, 2, 3, 4, 5, 8, 12, 16)[ri(0, 8)]
        hkv = ri(1, 4)
        h = hkv * n_rep
        b = ri(1, 5)
        q_lens = [ri(1, 150) for _ in range(b)]
        kv_lens = [max(1, ql + ri(-20, 100)) for ql in q_lens]
        causal, nsplit = bool(i % 3), (0, 1, 2, 5)[i % 4]
        if d == 128 and n_rep in (2, 4, 8):
            d = 64                                       # (that shape is the tuned kernel's, swept elsewhere)
        print(f"case {i}: d={d} h={h}/{hkv} kv={kv_lens} q={q_lens} causal={causal} nsplit={nsplit}", flush=True)
        args = _paged_case(b, h, hkv, d, kv_lens, q_lens, seed=7000 + i, holes=(i % 4 == 1))
        dev = [t.to(DEV) for t in args]
        qo, tb, ti = _cabi.paged_prefill_schedule(q_lens, DEV)
        mask = None
        if i % 2:
            w = max(kv_lens) + 3
            shape = [(b, w), (b, 1, max(q_lens), w), (b, h, max(q_lens), w), (b, h, 1, w)][(i // 2) % 4]
            mask = torch.rand(shape, generator=g) < 0.6
        got = _cabi.attn_paged_prefill(*dev, qo, tb, ti, mask=None if mask is None else mask.to(DEV),
                                       causal_offset=0 if causal else -1, nsplit=nsplit)
        _close(got, D.attn_paged_prefill(*args, qo.cpu(), causal=causal, mask=mask), f"sweep {i} prefill")
        m2 = None if mask is None else (torch.rand(b, max(kv_lens) + 3, generator=g) < 0.6)
        q1 = args[0][:b].contiguous()
        got = _cabi.attn_paged_decode(q1.to(DEV), *dev[1:], mask=None if m2 is None else m2.to(DEV), nsplit=nsplit)
        assert_bf16_close(got, D.attn_paged_decode(q1, *args[1:], mask=m2), what=f"sweep {i} decode")
