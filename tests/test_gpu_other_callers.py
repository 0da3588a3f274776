"""The other callers the ``aten::linear`` override intercepts besides the dense decoder's
projections: the router and the per-expert MLPs of a mixture-of-experts layer
(astrai/model/components/mlp.py:78-168) and the base / low-rank pair of a LoRA layer
(astrai/model/components/lora.py:31-54) -- many small weights, a handful of tokens per expert,
output widths of 8 .. 64 -- plus a traced module whose Linear goes through the custom ops
(the reference registers fake kernels for that, astrai/extension/ops/fp8.py:61-68,95-98).

Every intercepted Linear is checked against the oracle on its own inputs, and the kernel it
landed on is recorded (``astrai_w8a8_last_kernel``)."""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import w8a8_oracle as O
from tests.helpers import assert_bf16_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


class _Linear(nn.Module):   # components/linear.py:8-24
    def __init__(self, i, o, bias=False, std=0.02):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(o, i) * std)
        self.bias = nn.Parameter(torch.randn(o) * 0.1) if bias else None

    def forward(self, x):
        return F.linear(x, self.weight, self.bias)


class _MLP(nn.Module):      # components/mlp.py:23-43
    def __init__(self, dim, ffn):
        super().__init__()
        self.up, self.gate, self.down = _Linear(dim, ffn), _Linear(dim, ffn), _Linear(ffn, dim)

    def forward(self, x):
        return self.down(F.silu(self.gate(x)) * self.up(x))


class _MoE(nn.Module):      # components/mlp.py:78-168, inference path (no auxiliary loss)
    def __init__(self, dim, ffn, n_experts, k):
        super().__init__()
        self.k, self.e = k, n_experts
        self.router = _Linear(dim, n_experts, std=0.5)
        self.shared = _MLP(dim, ffn)
        self.experts = nn.ModuleList([_MLP(dim, ffn) for _ in range(n_experts)])

    def forward(self, x):
        shape = x.shape
        x = x.view(-1, shape[-1])
        probs = torch.softmax(self.router(x).float(), dim=-1).to(x.dtype)
        wts, idx = torch.topk(probs, self.k, dim=-1, sorted=False)
        wts = wts / wts.sum(dim=-1, keepdim=True)
        flat = idx.reshape(-1)
        sorted_experts, order = torch.sort(flat)
        tokens = x.repeat_interleave(self.k, dim=0)[order]
        weights = wts.reshape(-1, 1)[order]
        bounds = torch.cumsum(torch.bincount(sorted_experts, minlength=self.e), dim=0).tolist()
        out = torch.zeros_like(x)
        start = 0
        for e, end in enumerate(bounds):
            if end > start:
                out.index_add_(0, order[start:end] // self.k, self.experts[e](tokens[start:end]) * weights[start:end])
            start = end
        return (self.shared(x) + out).view(shape)


class _LoRA(nn.Module):     # components/lora.py:31-54
    def __init__(self, base, r, alpha=32):
        super().__init__()
        self.weight, self.bias = base.weight, base.bias
        self.scaling = alpha / r
        self.lora_A = nn.Parameter(torch.randn(r, base.weight.shape[1]) / r)
        self.lora_B = nn.Parameter(torch.randn(base.weight.shape[0], r) * 0.05)

    def forward(self, x):
        return F.linear(x, self.weight, self.bias) + (F.linear(x, self.lora_A) @ self.lora_B.T) * self.scaling


def _spy_linears(monkeypatch, policy_module, handler_name):
    """Record (x, w, bias, out, kernel) of every Linear the named policy handler takes."""
    from astrai_amd.extension import _cabi, dispatch
    calls = []
    inner = getattr(policy_module, handler_name)

    def spy(x, w, bias):
        out = inner(x, w, bias)
        if out is not None:
            calls.append((x.detach().clone(), w, bias, out.detach().clone(), _cabi.last_kernel()))
        return out

    patched = [spy if h is inner else h for h in dispatch._handlers]
    assert spy in patched
    monkeypatch.setattr(dispatch, "_handlers", patched)
    return calls


def test_moe_and_lora_linears_under_int8_autocast(monkeypatch):
    from astrai_amd.extension import w8a8
    torch.manual_seed(12)
    dim, ffn, n_exp = 512, 256, 8
    with torch.device(DEV):
        moe = _MoE(dim, ffn, n_exp, 2).to(torch.bfloat16).eval()
        loras = [_LoRA(_Linear(dim, 768, bias=True), r).to(torch.bfloat16).eval() for r in (8, 64)]
    x = torch.randn(3, 32, dim, device=DEV).to(torch.bfloat16)
    st = w8a8.int8_state()
    st.reset()
    calls = _spy_linears(monkeypatch, w8a8, "_int8_handler")
    quantized = []
    real_q = w8a8.quantize_int8_per_channel
    monkeypatch.setattr(w8a8, "quantize_int8_per_channel", lambda w: (quantized.append(tuple(w.shape)), real_q(w))[1])
    with torch.no_grad(), w8a8.int8_autocast(True):
        y = moe(x)
        first = len(calls)
        y2 = moe(x)
        outs = [m(x) for m in loras]
    n_weights = 1 + 3 + 3 * n_exp
    # one entry per weight, each quantized once although the layer ran twice
    assert len(st._weights) == n_weights + 2 * len(loras)
    assert len(quantized) == n_weights + 2 * len(loras)
    assert torch.equal(y, y2) and first >= 1 + 3 + 3 and len(calls) == 2 * first + 2 * len(loras)
    kernels = {}
    for xi, w, bias, out, kern in calls:
        wq, sw = O.int8_quantize_rows(w.detach().float().cpu().to(torch.bfloat16))
        want = O.int8_linear(xi.cpu(), wq, sw, None if bias is None else bias.detach().cpu())
        assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16)), (tuple(xi.shape), tuple(w.shape), kern)
        kernels.setdefault((xi.reshape(-1, xi.size(-1)).size(0) <= 128, kern), []).append(
            (xi.reshape(-1, xi.size(-1)).size(0), w.size(0), w.size(1)))
    print("kernels by (decode-sized M, family):", {k: sorted(set(v))[:6] for k, v in kernels.items()}, flush=True)
    # per-expert blocks (a few to a few dozen tokens) and the 96-token router / shared / LoRA calls
    # all run the weight-streaming decode kernels; nothing falls to the any-shape kernel
    assert {k[1] for k in kernels} <= {"gemv_dot", "gemv_rows"}, kernels.keys()
    for o in (y, *outs):
        assert torch.isfinite(o.float()).all() and o.float().abs().max() > 0
    st.reset()


def test_moe_and_lora_linears_under_fp8_autocast(monkeypatch):
    from astrai_amd.extension import fp8 as P
    torch.manual_seed(13)
    dim, ffn, n_exp = 512, 256, 8
    with torch.device(DEV):
        moe = _MoE(dim, ffn, n_exp, 2).to(torch.bfloat16).eval()
        lora = _LoRA(_Linear(dim, 768, bias=True), 16).to(torch.bfloat16).eval()
    x = torch.randn(2, 48, dim, device=DEV).to(torch.bfloat16)
    P.fp8_state().reset()
    calls = _spy_linears(monkeypatch, P, "_fp8_handler")
    with torch.no_grad(), P.fp8_autocast(True, recipe=P.DynamicScaling(), fp8_format="e4m3"):
        y = moe(x)
        z = lora(x)
    assert len(calls) >= 1 + 3 + 3 + 2
    seen = set()
    for xi, w, bias, out, kern in calls:
        x2, wc = xi.reshape(-1, xi.size(-1)).cpu(), w.detach().cpu()
        sx, sw = O.dynamic_scale(x2).reshape(1), O.dynamic_scale(wc).reshape(1)
        want = O.fp8_gemm(O.fp8_quantize(x2, sx, 0)[0], O.fp8_quantize(wc, sw, 0)[0], sx, sw)
        if bias is not None:
            want = want + bias.detach().cpu()        # dynamic scaling adds the bias in bf16 (fp8.py:299-301)
        assert_bf16_close(out.reshape(-1, w.size(0)), want, what=f"{tuple(x2.shape)} x {tuple(w.shape)} on {kern}")
        seen.add(kern)
    print("fp8 kernels:", sorted(seen), flush=True)
    assert seen <= {"gemv_rows_fp8"}, seen
    assert torch.isfinite(y.float()).all() and torch.isfinite(z.float()).all()
    P.fp8_state().reset()


def test_traced_module_runs_the_custom_ops():
    """torch.compile of a module whose Linear is written with the dispatcher ops
    custom::fp8_quantize / custom::fp8_gemm: the fake kernels give the tracer its shapes and the
    compiled module calls the HIP kernels (same bits as eager)."""
    from astrai_amd.extension.ops import fp8 as ops

    class QLinear(nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = nn.Parameter((torch.randn(384, 256) * 0.05).to(torch.bfloat16))
            self.register_buffer("sx", torch.tensor([4.0 / 448.0]))
            self.register_buffer("sw", torch.tensor([0.25 / 448.0]))

        def forward(self, x):
            x8, _ = ops.fp8_quantize(x, self.sx, 0)
            w8, _ = ops.fp8_quantize(self.weight, self.sw, 0)
            return ops.fp8_gemm(x8, w8, self.sx, self.sw)

    torch.manual_seed(3)
    m = QLinear().to(DEV).eval()
    x = torch.randn(40, 256, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        eager = m(x)
        ran = []
        for backend in ("aot_eager", "inductor"):
            torch._dynamo.reset()
            try:
                compiled = torch.compile(m, backend=backend, fullgraph=True)
                got = compiled(x)
            except Exception as e:   # no code generator for this backend on the box
                print(f"backend {backend} unavailable: {type(e).__name__}: {str(e)[:120]}", flush=True)
                continue
            assert got.shape == eager.shape and got.dtype == eager.dtype
            assert torch.equal(got, eager), backend
            ran.append(backend)
    torch._dynamo.reset()
    if not ran:
        pytest.skip("no torch.compile backend works on this box")
    want = O.fp8_gemm(O.fp8_quantize(x.cpu(), m.sx.cpu(), 0)[0], O.fp8_quantize(m.weight.detach().cpu(), m.sw.cpu(), 0)[0],
                      m.sx.cpu(), m.sw.cpu())
    assert_bf16_close(eager, want, what="traced linear")
