"""Benchmark of the quantized linear GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one launch of the pre-quantized fp8 e4m3fn per-tensor GEMM of
BASELINE config 1 (A[4096,4096] . B[4096,4096]^T, fp32 accumulate, bf16 out),
operands already resident in HBM. Prints ONE JSON line: the headline value is
that GEMM's TFLOP/s; `roofline` prices the same kernel against the dense fp8
MFMA peak; `cpu_baseline` is the CPU oracle timed on this host in the same run;
`extra` carries the other BASELINE shapes (int8 GEMM, decode GEMV GB/s, block
fp8, config 0 latency).
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA
PEAK_INT8_TOPS = 5000.0    # MI355X dense int8 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# HBM-side bytes per launch of the headline kernel from two counter passes
# (reads 101.7 MB + writes 34.4 MB); algorithmic bytes are 67.1 MB
HEADLINE_TRAFFIC_MB = 136.1
# share of the q|k|v, output, gate|up and down GEMV kernels in the kernel time of one fused
# config-4 decode layer (profiles/decoder_config4_int8_kernel_shares.txt)
DECODE_GEMV_SHARE = 0.49


LAUNCHES_PER_BATCH = 50   # event-timed launches per batch
TIMED_BATCHES = 7         # the reported duration is the median of this many batch averages
MAX_WARM_BATCHES = 60     # warm-up ends when two consecutive batches agree within 2% (or here)


def _timed_batch_ms(run_batch):
    """Duration of `run_batch()` (which launches on torch's current stream) by HIP events
    recorded on that stream."""
    import torch

    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    run_batch()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1)


def _protocol_us(run_batch, launches=LAUNCHES_PER_BATCH):
    """The fixed timing protocol of every kernel figure in the JSON line, whatever --steps
    and --warmup say: batches of `launches` back-to-back launches timed by HIP events;
    warm-up batches until two consecutive ones agree within 2% (at least two, i.e. >= 100
    launches); then the median of TIMED_BATCHES batch averages. Returns (microseconds per
    launch, {protocol details})."""
    import torch

    torch.cuda.synchronize()
    prev, warm = None, 0
    while warm < MAX_WARM_BATCHES:
        t = _timed_batch_ms(run_batch)
        warm += 1
        if prev is not None and abs(t - prev) <= 0.02 * prev:
            break
        prev = t
    ts = sorted(_timed_batch_ms(run_batch) for _ in range(TIMED_BATCHES))
    med = ts[len(ts) // 2]
    return med * 1e3 / launches, {"launches_per_batch": launches, "timed_batches": TIMED_BATCHES,
                                  "warm_batches": warm,
                                  "batch_spread": round((ts[-1] - ts[0]) / med, 4)}


def _kernel_us(fn):
    """_protocol_us for a host-launched kernel `fn`."""
    def batch():
        for _ in range(LAUNCHES_PER_BATCH):
            fn()
    return _protocol_us(batch)[0]


def _alternating_us(fns):
    """Same-run A/B of host-launched kernels: after the protocol's warm-up on each, timed
    batches alternate between them (a, b, a, b, ...), so that clock and temperature drift
    hits all alike; the median of TIMED_BATCHES batch averages each, in microseconds."""
    def batch_of(fn):
        def batch():
            for _ in range(LAUNCHES_PER_BATCH):
                fn()
        return batch

    batches = [batch_of(fn) for fn in fns]
    for b in batches:
        _protocol_us(b)
    ts = [[] for _ in fns]
    for _ in range(TIMED_BATCHES):
        for i, b in enumerate(batches):
            ts[i].append(_timed_batch_ms(b))
    return [sorted(t)[len(t) // 2] * 1e3 / LAUNCHES_PER_BATCH for t in ts]


def _graph_us(launch, n_launch=LAUNCHES_PER_BATCH):
    """_protocol_us with the batch captured in one HIP graph (`launch(i)` for i in
    range(n_launch)): removes host launch overhead for kernels of a few microseconds."""
    import torch

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for i in range(min(n_launch, 3)):
            launch(i)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for i in range(n_launch):
            launch(i)
    return _protocol_us(g.replay, n_launch)[0]


def _bench_decoder(dev):
    """BASELINE config 4: 24-layer GQA/SwiGLU decoder (hidden 2048, 16/4 heads, FFN 5632, vocab 32000),
    random-init bf16 weights quantized to int8 per channel, every Linear through the int8 kernels;
    batch 32 x 512-token prefill, then 128 greedy decode steps (eager and as a replayed HIP graph)."""
    import torch

    from astrai_amd.extension import w8a8
    from astrai_amd.model import (AutoRegressiveLM, AutoRegressiveLMConfig, DenseKVCache, fuse_int8_weights,
                                  greedy_generate, unfuse_int8_weights)

    cfg = AutoRegressiveLMConfig()
    torch.manual_seed(4)
    with torch.device(dev):
        model = AutoRegressiveLM(cfg).to(torch.bfloat16).eval()
    batch, prompt, steps = 32, 512, 128
    ids = torch.randint(0, cfg.vocab_size, (batch, prompt), generator=torch.Generator().manual_seed(4)).to(dev)
    w8a8.int8_state().reset()
    n_lin = w8a8.prepare_int8_weights(model)
    res = {"linears": n_lin, "batch": batch, "prompt_len": prompt, "decode_steps": steps}
    with torch.no_grad(), w8a8.int8_autocast(True):
        def prefill():
            cache = DenseKVCache(cfg, batch, prompt + steps, dev, torch.bfloat16)
            return model(ids, cache, torch.arange(prompt, device=dev))["logits"][:, -1].argmax(-1)

        for _ in range(2):
            prefill()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            prefill()
        torch.cuda.synchronize()
        t_pre = (time.perf_counter() - t0) / 3
        res["prefill_ms"] = round(t_pre * 1e3, 2)
        res["prefill_tokens_per_s"] = round(batch * prompt / t_pre)
        def decode_legs(prefix, t_prefill):
            for name, graph in (("eager", False), ("graph", True)):
                greedy_generate(model, ids, 8, use_graph=graph)  # warm
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                greedy_generate(model, ids, steps, use_graph=graph)
                torch.cuda.synchronize()
                t_all = time.perf_counter() - t0
                t_dec = max(t_all - t_prefill, 1e-9)
                res[f"{prefix}decode_{name}_ms_per_step"] = round(t_dec * 1e3 / (steps - 1), 3)
                res[f"{prefix}decode_{name}_tokens_per_s"] = round(batch * (steps - 1) / t_dec)

        decode_legs("", t_pre)
        # the same blocks with q|k|v and gate|up concatenated and the norm / SwiGLU
        # producers fused with the per-token quantizer
        res["fused_int8_matrices"] = fuse_int8_weights(model)
        for _ in range(2):
            prefill()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(3):
            prefill()
        torch.cuda.synchronize()
        t_pre_f = (time.perf_counter() - t0) / 3
        res["fused_prefill_ms"] = round(t_pre_f * 1e3, 2)
        res["fused_prefill_tokens_per_s"] = round(batch * prompt / t_pre_f)
        # GEMM share of the fused prefill, measured live: HIP events around every int8 product
        # (the four GEMM entries of a fused layer, their fused epilogues included, and the lm_head)
        from astrai_amd.extension import _cabi
        gemm_names = ("mm_int8", "mm_int8_resid", "mm_int8_swiglu", "mm_int8_rope_cache")
        real = {n: getattr(_cabi, n) for n in gemm_names}
        spans = []

        def timed(fn):
            def call(*a, **kw):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                out = fn(*a, **kw)
                e1.record()
                spans.append((e0, e1))
                return out
            return call

        for n in gemm_names:
            setattr(_cabi, n, timed(real[n]))
        try:
            w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            w0.record()
            prefill()
            w1.record()
            torch.cuda.synchronize()
        finally:
            for n in gemm_names:
                setattr(_cabi, n, real[n])
        in_gemm = sum(a.elapsed_time(b) for a, b in spans)
        res["gemm_share_of_gpu_time"] = {
            "fused_prefill": round(in_gemm / w0.elapsed_time(w1), 3),
            "fused_prefill_what": f"measured in this run: HIP events around the {len(spans)} int8 GEMM calls of one "
                                  "32 x 512-token prefill (q|k|v + rotary epilogue, output + residual, gate|up + "
                                  "SwiGLU epilogue and its one-read quantizer, down + residual, lm_head) over the "
                                  "events around the whole prefill",
            "fused_decode_step": DECODE_GEMV_SHARE,
            "fused_decode_step_what": "NOT measured in this run: share of the four weight-streaming GEMV kernels in "
                                      "the kernel time of a decode layer, from the rocprofv3 kernel trace in "
                                      "profiles/decoder_config4_int8_kernel_shares.txt (graph replays are not "
                                      "traced per kernel)"}
        decode_legs("fused_", t_pre_f)
        unfuse_int8_weights(model)
        # the same model with the stock bf16 kernels, for scale
    w8a8.int8_state().reset()
    with torch.no_grad():
        greedy_generate(model, ids, 8, use_graph=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        greedy_generate(model, ids, steps, use_graph=True)
        torch.cuda.synchronize()
        res["bf16_stock_total_ms_graph"] = round((time.perf_counter() - t0) * 1e3, 1)
    del model
    torch.cuda.empty_cache()
    return res


def _cpu_decoder_baseline(layers=1, prefill_batch=8, decode_steps=8):
    """BASELINE config 4 on the host CPU through the decoder oracle (every Linear the exact
    int8 oracle, dense cache), on a bounded sample: a `layers`-layer model of the config-4
    dimensions, the 512-token prefill of `prefill_batch` of the 32 sequences, then
    `decode_steps` greedy steps of all 32 (the cache of the prefilled sequences repeated).
    Rates are per token; the per-layer share (total minus the separately timed embedding +
    final norm + lm_head share) is scaled to 24 layers."""
    import torch
    import torch.nn.functional as F

    from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig
    from oracle import decoder_oracle as D

    threads = _cpu_threads()
    torch.set_num_threads(threads)
    cfg = AutoRegressiveLMConfig(num_hidden_layers=layers)
    full_layers = AutoRegressiveLMConfig().num_hidden_layers
    torch.manual_seed(4)
    model = AutoRegressiveLM(cfg).to(torch.bfloat16).eval()
    sd = {k: v.detach() for k, v in model.state_dict().items()}
    lin = D.int8_linear_fn(sd, fast=True)
    batch, prompt = 32, 512
    ids = torch.randint(0, cfg.vocab_size, (batch, prompt), generator=torch.Generator().manual_seed(4))
    ids = ids[:prefill_batch]
    hd = cfg.hidden_size // cfg.num_attention_heads
    kc = torch.zeros(layers, prefill_batch, cfg.num_key_value_heads, prompt + decode_steps, hd,
                     dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)

    def head(x_ids):   # what does not grow with the layer count
        x = F.embedding(x_ids, sd["embed_tokens.weight"])
        return lin(F.rms_norm(x, (cfg.hidden_size,), sd["norm.weight"], cfg.rms_norm_eps), "lm_head.weight")

    with torch.no_grad():
        D.forward_cached(sd, cfg, ids[:2, :64], lin, kc[:, :2], vc[:, :2], torch.arange(64))  # warm-up
        t0 = time.perf_counter()
        logits = D.forward_cached(sd, cfg, ids, lin, kc, vc, torch.arange(prompt))
        t_pre = time.perf_counter() - t0
        t0 = time.perf_counter()
        head(ids)
        t_pre_head = time.perf_counter() - t0
        rep = batch // prefill_batch
        tok = logits[:, -1].argmax(-1).reshape(-1, 1).repeat(rep, 1)
        kc, vc = kc.repeat(1, rep, 1, 1, 1), vc.repeat(1, rep, 1, 1, 1)
        del logits
        t0 = time.perf_counter()
        for i in range(decode_steps):
            lg = D.forward_cached(sd, cfg, tok, lin, kc, vc, torch.tensor([prompt + i]))
            tok = lg[:, -1].argmax(-1).reshape(batch, 1)
        t_dec = (time.perf_counter() - t0) / decode_steps
        t0 = time.perf_counter()
        for _ in range(decode_steps):
            head(tok)
        t_dec_head = (time.perf_counter() - t0) / decode_steps
    scale = full_layers / layers
    pre_full = (t_pre - t_pre_head) * scale + t_pre_head      # seconds for prefill_batch x 512 tokens
    dec_full = (t_dec - t_dec_head) * scale + t_dec_head
    return {"unit": "tokens/s", "cores": threads, "kind": "port",
            "prefill_tokens_per_s": round(prefill_batch * prompt / pre_full, 1),
            "decode_tokens_per_s": round(batch / dec_full, 1),
            "decode_ms_per_step_extrapolated_24_layers": round(dec_full * 1e3, 1),
            "measured": {"layers": layers, "prefill_sequences": prefill_batch, "prefill_s": round(t_pre, 2),
                         "prefill_head_share_s": round(t_pre_head, 2), "decode_ms_per_step": round(t_dec * 1e3, 1),
                         "decode_head_share_ms": round(t_dec_head * 1e3, 1)},
            "sample": f"EXTRAPOLATED: a {layers}-layer model of the config-4 dimensions; prefill of {prefill_batch} "
                      f"of the 32 x 512-token prompts and {decode_steps} decode steps of 32 sequences, timed once; "
                      f"layer share x {scale:g} + embedding / lm_head share"}


def _cpu_threads():
    """Threads the CPU baselines run on: the box's CPU share (16 for one GPU), which
    OMP_NUM_THREADS states there, never more than the logical CPUs present."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", "16")))
    except ValueError:
        n = min(n, 16)
    return max(1, min(n, 16))


def _host_info():
    """Logical CPUs, physical cores (distinct (package, core id) pairs of /proc/cpuinfo) and
    the CPU model of the host the CPU baselines ran on."""
    info = {"logical_cpus": os.cpu_count()}
    try:
        pairs, model, phys, core = set(), None, None, None
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name") and model is None:
                model = ln.split(":", 1)[1].strip()
            elif ln.startswith("physical id"):
                phys = ln.split(":", 1)[1].strip()
            elif ln.startswith("core id"):
                core = ln.split(":", 1)[1].strip()
            elif not ln.strip():
                if phys is not None and core is not None:
                    pairs.add((phys, core))
                phys = core = None
        info["physical_cores"] = len(pairs) or None
        info["cpu_model"] = model
    except OSError:
        pass
    return info


def _measured_ceilings():
    """What a kernel on this very GPU can approach, measured now: a register-resident
    loop of nothing but MFMAs on random operand bits (the power manager clocks it
    well below the datasheet rate) and a plain streaming read of a decode-size matrix.
    The micro-benchmark is a program of its own (astrai_amd/csrc/ubench), started as a
    child BEFORE this process touches the GPU, and not at all under a profiler (whose
    preloaded library has the GPU initialised already). Returns {} when it is not
    built or did not run."""
    exe = os.path.join(ROOT, "astrai_amd", "csrc", "ubench", "ceilings")
    if not os.access(exe, os.X_OK):
        return {}
    if "rocprof" in os.environ.get("LD_PRELOAD", "") or any(k.startswith("ROCPROF") for k in os.environ):
        return {}
    import re
    import subprocess
    try:
        out = subprocess.run([exe], capture_output=True, text=True, timeout=120, check=True).stdout
    except (OSError, subprocess.SubprocessError):
        return {}
    res = {}
    for key, pat in (("mfma_fp8_random_TFLOPs", r"mfma fp8 32x32x64\s+operands random:\s*([0-9.]+) Tops/s"),
                     ("mfma_fp8_16x16x128_random_TFLOPs", r"mfma fp8 16x16x128\s+operands random:\s*([0-9.]+) Tops/s"),
                     ("mfma_i8_random_TOPs", r"mfma i8 32x32x32\s+operands random:\s*([0-9.]+) Tops/s"),
                     ("hbm_stream_45MB_GBs", r"hbm read, 45.1 MB per launch[^:]*:\s*[0-9.]+ us per launch, ([0-9.]+) GB/s")):
        m = re.search(pat, out)
        if m:
            res[key] = float(m.group(1))
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--no-extra", action="store_true", help="headline kernel only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-model", action="store_true", help="skip the config-4 decoder leg")
    ap.add_argument("--decoder-trace", choices=["modular", "fused"], default=None,
                    help="tracing mode: build the config-4 decoder (Linear-by-Linear int8 path, or the fused "
                         "one), one prefill + 19 eager decode steps, nothing else")
    ap.add_argument("--trace-kernels", action="store_true",
                    help="tracing mode: a few launches of every auxiliary kernel (quantizers, policy-path "
                         "kernels, attention) at 4096 x 4096 / config-4 sizes, nothing else")
    ap.add_argument("--trace-gemms", action="store_true",
                    help="tracing mode: a few launches of the large GEMM kernels besides the headline one "
                         "(int8 4096^3, block-scaled config 3, fp8 with e4m3 output), nothing else")
    ap.add_argument("--pmc", action="store_true",
                    help="counter-collection mode: a few launches of the headline kernel and of a "
                         "plain 256 MiB device copy (the calibration kernel), nothing else")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the path: run with --gpus 1 "
                 "(no multi-GPU leg exists: the path shards by output columns or by K, one collective at most)")

    tracing = bool(args.decoder_trace or args.trace_kernels or args.trace_gemms or args.pmc)
    ceilings = {} if tracing else _measured_ceilings()

    import torch

    from astrai_amd.extension import _cabi

    if not torch.cuda.is_available():
        sys.exit("bench.py needs the MI355X (no CPU fallback exists)")
    lib = _cabi.load()
    if lib is None:
        sys.exit(f"HIP library missing: {_cabi.load_error()}")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream().cuda_stream

    def check(rc):
        if rc:
            raise RuntimeError(lib.astrai_w8a8_last_error().decode())

    if args.decoder_trace:
        from astrai_amd.extension import w8a8
        from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig, fuse_int8_weights, greedy_generate

        cfg = AutoRegressiveLMConfig()
        torch.manual_seed(4)
        with torch.device(dev):
            model = AutoRegressiveLM(cfg).to(torch.bfloat16).eval()
        ids = torch.randint(0, cfg.vocab_size, (32, 512), generator=torch.Generator().manual_seed(4)).to(dev)
        if args.decoder_trace == "fused":
            fuse_int8_weights(model)
        else:
            w8a8.prepare_int8_weights(model)
        with torch.no_grad(), w8a8.int8_autocast(True):
            greedy_generate(model, ids, 20, use_graph=False)
        torch.cuda.synchronize()
        print(json.dumps({"decoder_trace": args.decoder_trace, "prefill_tokens": 32 * 512, "decode_steps": 19}))
        return

    if args.trace_kernels:
        from astrai_amd.extension import get_module

        fp8m = get_module("fp8_mm")
        x = torch.randn(4096, 4096, device=dev).to(torch.bfloat16)
        s1 = torch.full((1,), 4.0 / 448.0, device=dev)
        hist, scale = torch.ones(16, device=dev), torch.ones(1, device=dev)
        b_, h_, hkv_, s_, n_ = 32, 16, 4, 512, 640
        q = torch.randn(b_, h_, s_, 128, device=dev).to(torch.bfloat16)
        kc = torch.randn(b_, hkv_, n_, 128, device=dev).to(torch.bfloat16)
        vc = torch.randn(b_, hkv_, n_, 128, device=dev).to(torch.bfloat16)
        pos = torch.arange(s_, device=dev)
        q1 = q[:, :, -1:].contiguous()
        last = torch.tensor([n_ - 1], device=dev)
        k_pool = kc.permute(0, 2, 1, 3).reshape(b_ * n_, hkv_, 128).contiguous()
        v_pool = vc.permute(0, 2, 1, 3).reshape(b_ * n_, hkv_, 128).contiguous()
        table = torch.randperm(b_ * n_, device=dev).int().reshape(b_, n_).contiguous()
        rows = torch.arange(b_, dtype=torch.int32, device=dev)
        indptr = (torch.arange(b_ + 1, device=dev) * n_).int()
        # the reference-facing attention entries: ragged paged prefill (tuned kernel, with and without a
        # mask tensor), the same workload at head_dim 64 on the general kernel, rotary embedding
        qp = q.permute(0, 2, 1, 3).reshape(b_ * s_, h_, 128).contiguous()
        qo, tb, ti = _cabi.paged_prefill_schedule([s_] * b_, dev)
        key_mask = torch.ones(b_, n_, dtype=torch.bool, device=dev)
        q64 = torch.randn(b_ * s_, 2 * h_, 64, device=dev).to(torch.bfloat16)
        k64 = torch.randn(b_ * n_, 2 * hkv_, 64, device=dev).to(torch.bfloat16)
        v64 = torch.randn(b_ * n_, 2 * hkv_, 64, device=dev).to(torch.bfloat16)
        freqs = torch.randn(b_ * s_, 64, 2, device=dev)
        for _ in range(5):
            _cabi.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, tb, ti, causal_offset=0)
            _cabi.attn_paged_prefill(qp, k_pool, v_pool, table, rows, indptr, qo, tb, ti, mask=key_mask,
                                     causal_offset=0)
            _cabi.attn_paged_prefill(q64, k64, v64, table, rows, indptr, qo, tb, ti, causal_offset=0)
            _cabi.attn_paged_decode(q64[:b_].contiguous(), k64, v64, table, rows, indptr)
            _cabi.rotary_emb(qp, freqs)
        for _ in range(5):
            x8, amax = fp8m.quantize_bf16(x, s1, 0)                    # quantize_fp8_kernel
            fp8m.quantize_transpose_bf16(x, s1, 0, True, True)         # quantize_transpose_fp8_kernel
            fp8m.amax_bf16(x)                                          # amax_bf16_kernel
            fp8m.amax_ring_push(hist, 3, amax, scale, 448.0, 1.0)      # amax_ring_push_kernel
            _cabi.quantize_int8_rows(x)                                # quantize_int8_rows_kernel
            _cabi.attn_prefill(q, kc, vc, pos)                         # attn_prefill_kernel
            _cabi.attn_decode(q1, kc, vc, last)                        # attn_decode_partial/merge (dense)
            _cabi.attn_paged_decode(q1.reshape(b_, h_, 128), k_pool, v_pool, table, rows, indptr)
        torch.cuda.synchronize()
        print(json.dumps({"trace_kernels": "5 launches each; sizes: 4096x4096 bf16 for the quantizers, "
                                           "32 x 16/4 heads x 512 new tokens x 128 for prefill attention, "
                                           "32 sequences x 640 keys for decode attention"}))
        return

    if args.trace_gemms:
        xq = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device=dev)
        wq = torch.randint(-127, 128, (4096, 4096), dtype=torch.int8, device=dev)
        sx, sw = torch.rand(4096, device=dev) + 0.5, torch.rand(4096, device=dev) + 0.5
        y = torch.empty(4096, 4096, device=dev, dtype=torch.bfloat16)
        # config 3 data (seed 3, 1% x20 outliers in the weight), quantized on the device
        g3 = torch.Generator().manual_seed(3)   # activation, weight, outlier mask, in this order
        x3 = torch.randn(8192, 7168, generator=g3).to(torch.bfloat16)
        w3 = torch.randn(2048, 7168, generator=g3) * 0.02
        w3 = torch.where(torch.rand(2048, 7168, generator=g3) < 0.01, w3 * 20.0, w3).to(torch.bfloat16)
        a3, sa3 = _cabi.quantize_fp8_block128_act(x3.to(dev))
        b3, sb3 = _cabi.quantize_fp8_block128_weight(w3.to(dev))
        y3 = torch.empty(8192, 2048, device=dev, dtype=torch.bfloat16)
        a8 = (torch.randn(4096, 4096, device=dev) * 0.5).to(torch.float8_e4m3fn)
        b8 = (torch.randn(4096, 4096, device=dev) * 0.5).to(torch.float8_e4m3fn)
        one = torch.ones(1, device=dev)
        y8 = torch.empty(4096, 4096, device=dev, dtype=torch.float8_e4m3fn)
        for _ in range(20):
            check(lib.astrai_w8a8_gemm_int8_ptpc(xq.data_ptr(), wq.data_ptr(), sx.data_ptr(), sw.data_ptr(), None,
                                                 y.data_ptr(), 4096, 4096, 4096, 0, stream))
            check(lib.astrai_w8a8_gemm_fp8_block128(a3.data_ptr(), b3.data_ptr(), sa3.data_ptr(), sb3.data_ptr(),
                                                    None, y3.data_ptr(), 8192, 2048, 7168, stream))
            check(lib.astrai_w8a8_gemm_fp8_pt(a8.data_ptr(), b8.data_ptr(), one.data_ptr(), one.data_ptr(),
                                              one.data_ptr(), None, y8.data_ptr(), 4096, 4096, 4096, 0, 1, stream))
        # token blocks between decode and full prefill on the config-4 projections (128 x 128 tiles)
        mids = []
        for (mm, nn, kk) in ((2048, 3072, 2048), (2048, 2048, 5632), (1024, 11264, 2048)):
            mx = (torch.randn(mm, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            mw = (torch.randn(nn, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            mids.append((mx, mw, torch.rand(mm, device=dev) + 0.5, torch.rand(nn, device=dev) + 0.5,
                         torch.empty(mm, nn, device=dev, dtype=torch.bfloat16), mm, nn, kk))
        for _ in range(20):
            for (mx, mw, msx, msw, my, mm, nn, kk) in mids:
                check(lib.astrai_w8a8_gemm_int8_ptpc(mx.data_ptr(), mw.data_ptr(), msx.data_ptr(), msw.data_ptr(),
                                                     None, my.data_ptr(), mm, nn, kk, 0, stream))
        # block-scaled shapes below the large-tile kernel: a mid-size block of tokens and a decode step on
        # config-3-like weights; then an int8 product with four token rows past whole 256-row tiles
        xb = torch.randn(1024, 4096, device=dev).to(torch.bfloat16)
        wb = torch.randn(11008, 4096, device=dev).to(torch.bfloat16) * 0.02
        ab, sab = _cabi.quantize_fp8_block128_act(xb)
        bb, sbb = _cabi.quantize_fp8_block128_weight(wb)
        yb = torch.empty(1024, 11008, device=dev, dtype=torch.bfloat16)
        a3d, sa3d = a3[:16].contiguous(), sa3[:16].contiguous()
        xt = torch.randint(-127, 128, (4100, 4096), dtype=torch.int8, device=dev)
        sxt = torch.rand(4100, device=dev) + 0.5
        yt = torch.empty(4100, 4096, device=dev, dtype=torch.bfloat16)
        for _ in range(20):
            check(lib.astrai_w8a8_gemm_fp8_block128(ab.data_ptr(), bb.data_ptr(), sab.data_ptr(), sbb.data_ptr(),
                                                    None, yb.data_ptr(), 1024, 11008, 4096, stream))
            check(lib.astrai_w8a8_gemm_fp8_block128(a3d.data_ptr(), b3.data_ptr(), sa3d.data_ptr(), sb3.data_ptr(),
                                                    None, y3.data_ptr(), 16, 2048, 7168, stream))
            check(lib.astrai_w8a8_gemm_int8_ptpc(xt.data_ptr(), wq.data_ptr(), sxt.data_ptr(), sw.data_ptr(), None,
                                                 yt.data_ptr(), 4100, 4096, 4096, 0, stream))
        # a few hundred tokens: 64 x 64 tiles behind a ring of stages (int8, two shapes in turn)
        fews = []
        for (mm, nn, kk) in ((256, 4096, 4096), (384, 2048, 5632)):
            mx = (torch.randn(mm, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            mw = (torch.randn(nn, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            fews.append((mx, mw, torch.rand(mm, device=dev) + 0.5, torch.rand(nn, device=dev) + 0.5,
                         torch.empty(mm, nn, device=dev, dtype=torch.bfloat16), mm, nn, kk))
        for _ in range(20):
            for (mx, mw, msx, msw, my, mm, nn, kk) in fews:
                check(lib.astrai_w8a8_gemm_int8_ptpc(mx.data_ptr(), mw.data_ptr(), msx.data_ptr(), msw.data_ptr(),
                                                     None, my.data_ptr(), mm, nn, kk, 0, stream))
        torch.cuda.synchronize()
        print(json.dumps({"trace_gemms": "20 launches each: int8 4096^3 per-token x per-channel (bf16 out), fp8 "
                                         "128-block 8192x2048x7168 on config-3 data, fp8 4096^3 with e4m3 output; "
                                         "then int8 2048x3072x2048, 2048x2048x5632, 1024x11264x2048 (mid-size kernel); "
                                         "then block-scaled 1024x11008x4096 (mid-size kernel) and 16x2048x7168 "
                                         "(row-range kernel), and int8 4100x4096x4096 (large tiles + a four-row tail); "
                                         "then int8 256x4096x4096 and 384x2048x5632 (small-tile kernel)"}))
        return

    # ---------------- headline: config 1, fp8 per-tensor 4096^3 ----------------
    M = N = K = 4096
    g = torch.Generator().manual_seed(1)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    b = torch.randn(N, K, generator=g).to(torch.bfloat16)
    sa = (a.abs().amax().float() / 448.0).reshape(1)
    sb = (b.abs().amax().float() / 448.0).reshape(1)
    a8_cpu = (a.float() / sa).to(torch.float8_e4m3fn)
    b8_cpu = (b.float() / sb).to(torch.float8_e4m3fn)
    a8, b8 = a8_cpu.to(dev), b8_cpu.to(dev)
    sa_d, sb_d = sa.to(dev), sb.to(dev)
    out = torch.empty(M, N, device=dev, dtype=torch.bfloat16)

    def step():
        check(lib.astrai_w8a8_gemm_fp8_pt(a8.data_ptr(), b8.data_ptr(), sa_d.data_ptr(),
                                          sb_d.data_ptr(), None, None, out.data_ptr(),
                                          M, N, K, 0, 0, stream))

    if args.pmc:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            step()
        for _ in range(3):
            dst.copy_(src)
        # decode GEMV (config 2 shape) over four distinct weight buffers, after the
        # 512 MiB of copy traffic above has pushed everything else out of the caches
        gn, gk = 11008, 4096
        ring = [torch.randint(-127, 128, (gn, gk), dtype=torch.int8, device=dev) for _ in range(4)]
        gsw = torch.rand(gn, device=dev) + 0.5
        dst.copy_(src)
        gemv_ms = (1, 4, 16, 64)
        for gm in gemv_ms:
            gx = torch.randint(-127, 128, (gm, gk), dtype=torch.int8, device=dev)
            gsx = torch.rand(gm, device=dev) + 0.5
            gy = torch.empty(gm, gn, device=dev, dtype=torch.bfloat16)
            for w in ring:
                check(lib.astrai_w8a8_gemv_int8_ptpc(gx.data_ptr(), w.data_ptr(), gsx.data_ptr(), gsw.data_ptr(),
                                                     None, gy.data_ptr(), gm, gn, gk, 0, stream))
        # the same four buffers read as e4m3fn codes by the fp8 instance of the row-range kernel
        # (arbitrary bytes, NaN codes included: only time and traffic are of interest here)
        one = torch.ones(1, device=dev)
        for gm in gemv_ms:
            gx8 = torch.randint(-127, 128, (gm, gk), dtype=torch.int8, device=dev)
            gy = torch.empty(gm, gn, device=dev, dtype=torch.bfloat16)
            for w in ring:
                check(lib.astrai_w8a8_gemm_fp8_pt(gx8.data_ptr(), w.data_ptr(), one.data_ptr(), one.data_ptr(),
                                                  None, None, gy.data_ptr(), gm, gn, gk, 0, 0, stream))
        torch.cuda.synchronize()
        print(json.dumps({"pmc_mode": True, "gemm_launches": 5, "copy_launches": 4,
                          "copy_bytes_each_way": 256 << 20,
                          "gemm_algorithmic_bytes": 2 * M * K + 2 * M * N,
                          "gemv_launches": "4 each at M = 1 (dot kernel), 4, 16, 64 (rows kernel), 11008x4096, "
                                           "every launch on another 45 MB weight buffer; then the same 16 launches "
                                           "of the fp8 rows kernel",
                          "gemv_algorithmic_bytes": {f"M{m}": gn * gk + m * gk + 2 * m * gn + 4 * gn + 4 * m
                                                     for m in gemv_ms}}))
        return

    flop = 2.0 * M * N * K
    # the kernel's own time first (fixed protocol, see `roofline.timing`), so that the driver's
    # --warmup / --steps below find the GPU at its working clocks, not coming out of idle
    def step_batch():
        for _ in range(LAUNCHES_PER_BATCH):
            step()

    kern_us, proto = _protocol_us(step_batch)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = flop / (ms_per_step * 1e-3) / 1e12

    achieved = flop / (kern_us * 1e-6) / 1e12
    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP8_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_FP8_TFLOPS, 4),
                "traffic": HEADLINE_TRAFFIC_MB, "traffic_unit": "MB per launch; NOT measured in this run: "
                "rocprofv3 FETCH_SIZE + WRITE_SIZE of this kernel, calibrated on a plain copy, from "
                "profiles/gemm_fp8_wave128_q16_4096cubed.txt",
                "kernel": "gemm_wave128_q16_kernel<e4m3,per-tensor> (256x256x128 tiles, 4 waves, v_mfma_f32_16x16x128_f8f6f4)",
                "avg_launch_us": round(kern_us, 2),
                "timing": {"what": "HIP events on the launch stream; median of batch averages after a warm-up "
                                   "that ends when two consecutive batches agree within 2%; independent of "
                                   "--steps / --warmup, and run before them", **proto}}
    if "mfma_fp8_16x16x128_random_TFLOPs" in ceilings:
        # the same kernel against what this GPU's MFMA pipe sustains on random operand bits
        roofline["measured_ceiling"] = {
            "value": ceilings["mfma_fp8_16x16x128_random_TFLOPs"], "unit": "TFLOP/s",
            "frac": round(achieved / ceilings["mfma_fp8_16x16x128_random_TFLOPs"], 4),
            "what": "register-resident v_mfma_f32_16x16x128_f8f6f4 loop (the kernel's instruction), random "
                    "operand bits, measured in this run"}

    # ---------------- CPU baseline: the oracle on this host ----------------
    cpu_baseline = None
    if not args.no_cpu:
        from oracle import w8a8_oracle as O

        cores = _cpu_threads()
        torch.set_num_threads(cores)
        O.fp8_gemm(a8_cpu[:256], b8_cpu, sa, sb)  # warm-up
        trials = []
        for _ in range(3):
            t0 = time.perf_counter()
            O.fp8_gemm(a8_cpu, b8_cpu, sa, sb)
            trials.append(time.perf_counter() - t0)
        med = sorted(trials)[1]
        cpu_baseline = {"value": round(flop / med / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
                        "kind": "port",
                        "sample": "full config-1 GEMM (4096^3, fp8 upcast + fp32 matmul + scale -> bf16), "
                                  "median of 3 after 1 warm-up", "ms": round(med * 1e3, 1)}

    extra = {}
    cpu_more = {}
    if not args.no_extra:
        def ms_of(fn):
            return _kernel_us(fn) * 1e-3

        def cpu_median_ms(fn, trials=3):
            fn()  # warm-up
            ts = []
            for _ in range(trials):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return sorted(ts)[len(ts) // 2] * 1e3

        # ---- the vendor library's fp8 GEMM on the same config-1 tensors (torch._scaled_mm), a
        # labelled comparator: alternating batches with this repository's kernel in the same run
        try:
            b8_t = b8.t()
            out_v = torch._scaled_mm(a8, b8_t, scale_a=sa_d, scale_b=sb_d, out_dtype=torch.bfloat16)

            def step_vendor():
                torch._scaled_mm(a8, b8_t, scale_a=sa_d, scale_b=sb_d, out_dtype=torch.bfloat16, out=out_v)

            try:
                step_vendor()
            except (RuntimeError, TypeError):
                def step_vendor():  # noqa: F811  (no out= on this build: the allocation is cached)
                    torch._scaled_mm(a8, b8_t, scale_a=sa_d, scale_b=sb_d, out_dtype=torch.bfloat16)
            ours_us, vendor_us = _alternating_us([step, step_vendor])
            extra["fp8_gemm_4096_vendor_comparator"] = {
                "what": "torch._scaled_mm (the vendor library's fp8 GEMM; not used by the product) on the same "
                        "config-1 operands and steps, bf16 out; alternating batches of 50 launches with "
                        "astrai_w8a8_gemm_fp8_pt, median of 7 each",
                "this_kernel_us": round(ours_us, 2), "scaled_mm_us": round(vendor_us, 2),
                "this_over_vendor": round(ours_us / vendor_us, 4)}
            del out_v
        except (RuntimeError, NotImplementedError, AttributeError) as e:
            extra["fp8_gemm_4096_vendor_comparator"] = {"unavailable": str(e)[:200]}

        # ---- int8 4096^3 through the tiled kernel: operands drawn like config 0 (seeded bf16
        # N(0,1) activations and N(0,0.02) weights, quantized per token / per channel on the device)
        gi = torch.Generator().manual_seed(0)
        xi = torch.randn(M, K, generator=gi).to(torch.bfloat16).to(dev)
        wi = (torch.randn(N, K, generator=gi) * 0.02).to(torch.bfloat16).to(dev)
        ai, sxi = _cabi.quantize_int8_rows(xi)
        bi, swi = _cabi.quantize_int8_rows(wi)
        sxi, swi = sxi.reshape(-1).contiguous(), swi.reshape(-1).contiguous()
        del xi, wi

        def step_i8():
            check(lib.astrai_w8a8_gemm_int8_ptpc_tiled(ai.data_ptr(), bi.data_ptr(), sxi.data_ptr(),
                                                       swi.data_ptr(), None, out.data_ptr(),
                                                       M, N, K, 0, stream))

        ms = ms_of(step_i8)
        tops = flop / (ms * 1e-3) / 1e12
        extra["int8_gemm_4096"] = {"data": "seed 0, bf16 N(0,1) x N(0,0.02) quantized per token / per channel",
                                   "us": round(ms * 1e3, 2), "TOP/s": round(tops, 1),
                                   "frac_mfma_peak": round(tops / PEAK_INT8_TOPS, 4)}

        # ---- fp8 per-tensor with bias epilogue
        bias = (torch.randn(N) * 0.1).to(torch.bfloat16).to(dev)

        def step_bias():
            check(lib.astrai_w8a8_gemm_fp8_pt(a8.data_ptr(), b8.data_ptr(), sa_d.data_ptr(),
                                              sb_d.data_ptr(), None, bias.data_ptr(), out.data_ptr(),
                                              M, N, K, 0, 0, stream))

        ms = ms_of(step_bias)
        extra["fp8_gemm_4096_bias"] = {"us": round(ms * 1e3, 2),
                                       "TFLOP/s": round(flop / (ms * 1e-3) / 1e12, 1)}
        del ai, bi

        # ---- fp8 with one scale per activation row and per weight row
        sa_rows = sa_d.expand(M).contiguous()
        sb_rows = sb_d.expand(N).contiguous()

        def step_rowcol():
            check(lib.astrai_w8a8_gemm_fp8_ptpc(a8.data_ptr(), b8.data_ptr(), sa_rows.data_ptr(),
                                                sb_rows.data_ptr(), None, out.data_ptr(), M, N, K, 0, stream))

        ms = ms_of(step_rowcol)
        extra["fp8_gemm_4096_row_and_column_scales"] = {"us": round(ms * 1e3, 2),
                                                        "TFLOP/s": round(flop / (ms * 1e-3) / 1e12, 1)}

        # ---- fp8 linear backward at 4096^3 (dX and dW GEMMs + the three transposing
        # quantizer passes), through the module the registry hands out
        from astrai_amd.extension import get_module

        mod = get_module("fp8_mm")
        gb16 = torch.randn(M, N, device=dev).to(torch.bfloat16)
        xb16 = torch.randn(M, K, device=dev).to(torch.bfloat16)
        wb16 = torch.randn(N, K, device=dev).to(torch.bfloat16)
        s_one = torch.full((1,), 4.0 / 448.0, device=dev)

        def step_bwd():
            mod.linear_backward_fp8(gb16, xb16, wb16, [1, 1, 0], s_one, s_one, s_one, 0)

        ms = ms_of(step_bwd)

        def step_qt():
            mod.quantize_transpose_bf16(gb16, s_one, 0, True, True)

        ms_qt = ms_of(step_qt)
        extra["fp8_linear_backward_4096"] = {
            "us": round(ms * 1e3, 1), "TFLOP/s_two_gemms": round(2 * flop / (ms * 1e-3) / 1e12, 1),
            "quantize_transpose_us": round(ms_qt * 1e3, 2),
            "quantize_transpose_GB/s": round(M * N * 4 / (ms_qt * 1e-3) / 1e9, 0)}
        # ---- the whole Linear as the dispatcher override runs it (measure / quantize /
        # GEMM / ring update), per recipe, with and without the opt-in weight-code cache
        import torch.nn.functional as F
        from astrai_amd.extension import fp8 as P

        e2e = {"bf16_stock_us": round(ms_of(lambda: F.linear(xb16, wb16)) * 1e3, 1),
               "what": "F.linear(x, w) at 4096^3 under fp8_autocast; `_us` is the default (the weight's codes "
                       "are kept while it is unmodified, since it takes no gradient here), "
                       "`_requantized_weight_us` with fp8_cache_weights(False): the weight measured / "
                       "quantized in every call, as in a training step"}
        for rname, recipe in (("dynamic", P.DynamicScaling()), ("delayed", P.DelayedScaling())):
            for cache in (False, None):
                P.fp8_state().reset()
                with P.fp8_autocast(True, recipe=recipe):
                    P.fp8_cache_weights(cache)
                    ms = ms_of(lambda: F.linear(xb16, wb16))
                e2e[f"{rname}{'_requantized_weight' if cache is False else ''}_us"] = round(ms * 1e3, 1)
        P.fp8_state().reset()
        extra["fp8_linear_4096_through_dispatcher"] = e2e
        del gb16, xb16, wb16

        # ---- config 3: block-scaled fp8 8192 x 2048 x 7168 on the seed-3 tensors (activation,
        # weight, outlier mask drawn in this order; 1% of the weights x 20), quantized per
        # 1x128 / 128x128 block by the device quantizers
        M3, N3, K3 = 8192, 2048, 7168
        g3 = torch.Generator().manual_seed(3)
        x3 = torch.randn(M3, K3, generator=g3).to(torch.bfloat16)
        w3 = torch.randn(N3, K3, generator=g3) * 0.02
        w3 = torch.where(torch.rand(N3, K3, generator=g3) < 0.01, w3 * 20.0, w3).to(torch.bfloat16)
        a3, sa3 = _cabi.quantize_fp8_block128_act(x3.to(dev))
        b3, sb3 = _cabi.quantize_fp8_block128_weight(w3.to(dev))
        out3 = torch.empty(M3, N3, device=dev, dtype=torch.bfloat16)

        def step_blk():
            check(lib.astrai_w8a8_gemm_fp8_block128(a3.data_ptr(), b3.data_ptr(), sa3.data_ptr(),
                                                    sb3.data_ptr(), None, out3.data_ptr(),
                                                    M3, N3, K3, stream))

        ms = ms_of(step_blk)
        f3 = 2.0 * M3 * N3 * K3
        extra["fp8_block128_8192x2048x7168"] = {
            "data": "BASELINE config 3 (seed 3)",
            "us": round(ms * 1e3, 2), "TFLOP/s": round(f3 / (ms * 1e-3) / 1e12, 1),
            "frac_mfma_peak": round(f3 / (ms * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4)}
        if not args.no_cpu:
            from oracle import w8a8_oracle as O

            # CPU: the first 1024 activation rows (1/8 of the GEMM), scaled to the whole
            rows = 1024
            a3c, sa3c = a3[:rows].cpu(), sa3[:rows].cpu()
            b3c, sb3c = b3.cpu(), sb3.cpu()
            cms = cpu_median_ms(lambda: O.fp8_gemm_blockscaled(a3c, b3c, sa3c, sb3c))
            cpu_more["config3_fp8_block128"] = {
                "value": round(f3 * rows / M3 / (cms * 1e-3) / 1e12, 4), "unit": "TFLOP/s", "cores": _cpu_threads(),
                "kind": "port", "ms_sample": round(cms, 1), "ms_whole_extrapolated": round(cms * M3 / rows, 1),
                "sample": f"rows 0..{rows - 1} of the config-3 activation against the whole weight (1/8 of the "
                          "GEMM: 56 K-block fp32 matmuls with the block steps applied), median of 3 after 1 warm-up"}
            del a3c, b3c
        del a3, b3, out3, x3, w3

        # ---- config-4 prefill MLP entry: gate|up projection + SwiGLU + per-token int8, as one GEMM
        # with the product in its epilogue + the one-read quantizer, against GEMM + producer kernel
        Mg, Wg, Kg = 32 * 512, 5632, 2048
        gsw = torch.Generator().manual_seed(4)
        xg = torch.randn(Mg, Kg, generator=gsw).to(torch.bfloat16).to(dev)
        wgate = (torch.randn(Wg, Kg, generator=gsw) * 0.02).to(torch.bfloat16).to(dev)
        wup = (torch.randn(Wg, Kg, generator=gsw) * 0.02).to(torch.bfloat16).to(dev)
        xq, sxq = _cabi.quantize_int8_rows(xg)
        (wgq, sgq), (wuq, suq) = _cabi.quantize_int8_rows(wgate), _cabi.quantize_int8_rows(wup)
        sxq, sgq, suq = sxq.reshape(-1), sgq.reshape(-1), suq.reshape(-1)
        wcat, scat = torch.cat((wgq, wuq)), torch.cat((sgq, suq))
        wblk, sblk = _cabi.swiglu_block_rows(wgq, wuq), _cabi.swiglu_block_rows(sgq, suq)

        def step_chain():
            gu = _cabi.mm_int8(xq, wcat, sxq, scat)
            _cabi.silu_mul_quantize_int8(gu[:, :Wg], gu[:, Wg:])

        ms_chain = ms_of(step_chain)
        ms_fused = ms_of(lambda: _cabi.mm_int8_swiglu(xq, wblk, sxq, sblk, fused=True))
        extra["int8_gate_up_swiglu_16384x11264x2048"] = {
            "data": "config-4 prefill shape, N(0,1) activations, N(0,0.02) weights, seed 4",
            "gemm_plus_producer_us": round(ms_chain * 1e3, 1),
            "swiglu_epilogue_gemm_plus_quantizer_us": round(ms_fused * 1e3, 1),
            "TOP/s_of_the_fused_pair": round(2.0 * Mg * 2 * Wg * Kg / (ms_fused * 1e-3) / 1e12, 1)}
        del xg, wgate, wup, xq, wgq, wuq, wcat, wblk

        # ---- token blocks between decode and full prefill on the config-4 projections: too few
        # 256 x 256 tiles for the chip, 128 x 128 tiles instead (N(0, 32) codes, per-token x per-channel)
        mid = {}
        for (mm, nn, kk) in ((2048, 3072, 2048), (2048, 2048, 5632), (1024, 11264, 2048)):
            mx = (torch.randn(mm, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            mw = (torch.randn(nn, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            msx, msw = torch.rand(mm, device=dev) + 0.5, torch.rand(nn, device=dev) + 0.5
            my = torch.empty(mm, nn, device=dev, dtype=torch.bfloat16)
            ms_mid = ms_of(lambda: check(lib.astrai_w8a8_gemm_int8_ptpc(
                mx.data_ptr(), mw.data_ptr(), msx.data_ptr(), msw.data_ptr(), None, my.data_ptr(), mm, nn, kk, 0,
                stream)))
            mid[f"{mm}x{nn}x{kk}"] = {"us": round(ms_mid * 1e3, 2),
                                      "TOP/s": round(2.0 * mm * nn * kk / (ms_mid * 1e-3) / 1e12, 1)}
            del mx, mw, my
        extra["int8_gemm_token_blocks_128x128_tiles"] = mid

        # ---- a few hundred tokens against the config-4 projections (a short prompt, a large decode
        # batch): too few 128 x 128 tiles as well; 64 x 64 tiles behind a ring of direct-to-LDS stages
        few = {}
        for (mm, nn, kk) in ((256, 3072, 2048), (256, 2048, 5632), (384, 2048, 5632), (256, 4096, 4096)):
            mx = (torch.randn(mm, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            mw = (torch.randn(nn, kk, device=dev) * 32).clamp(-127, 127).round().to(torch.int8)
            msx, msw = torch.rand(mm, device=dev) + 0.5, torch.rand(nn, device=dev) + 0.5
            my = torch.empty(mm, nn, device=dev, dtype=torch.bfloat16)
            ms_few = ms_of(lambda: check(lib.astrai_w8a8_gemm_int8_ptpc(
                mx.data_ptr(), mw.data_ptr(), msx.data_ptr(), msw.data_ptr(), None, my.data_ptr(), mm, nn, kk, 0,
                stream)))
            few[f"{mm}x{nn}x{kk}"] = {"us": round(ms_few * 1e3, 2),
                                      "TOP/s": round(2.0 * mm * nn * kk / (ms_few * 1e-3) / 1e12, 1),
                                      "kernel": _cabi.last_kernel()}
            del mx, mw, my
        extra["int8_gemm_few_hundred_tokens_64x64_tiles"] = few

        # ---- config 2: decode GEMV on the seed-2 tensors (activation and weight quantized per
        # token / per channel by the oracle's quantizer on the host), weights rotated through a
        # ring of ten copies (451 MB) so that the 256 MB Infinity Cache cannot serve them
        from oracle import w8a8_oracle as O2

        N2, K2 = 11008, 4096
        x2_all, w2, _ = O2.make_inputs(2, 64, N2, K2)
        wq2, sw2c = O2.int8_quantize_rows(w2)
        ring = [wq2.to(dev).clone() for _ in range(10)]
        sw2 = sw2c.reshape(-1).to(dev)
        gemv, cpu_c2 = {}, {}
        for m in (1, 4, 16, 64):
            xq2c, sx2c = O2.int8_quantize_rows(x2_all[:m])
            x2, sx2 = xq2c.to(dev), sx2c.reshape(-1).to(dev)
            y2 = torch.empty(m, N2, device=dev, dtype=torch.bfloat16)

            def launch(i, x2=x2, sx2=sx2, y2=y2, m=m):
                w = ring[i % len(ring)]
                check(lib.astrai_w8a8_gemm_int8_ptpc(
                    x2.data_ptr(), w.data_ptr(), sx2.data_ptr(), sw2.data_ptr(), None,
                    y2.data_ptr(), m, N2, K2, 0, torch.cuda.current_stream().cuda_stream))

            us = _graph_us(launch)
            nbytes = N2 * K2 + m * K2 + 2 * m * N2 + 4 * N2 + 4 * m
            gbs = nbytes / (us * 1e-6) / 1e9
            us1 = _graph_us(lambda i: launch(0))
            gemv[f"M{m}"] = {"us": round(us, 2), "GB/s": round(gbs, 0),
                             "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                             **({"frac_measured_stream": round(gbs / ceilings["hbm_stream_45MB_GBs"], 4)}
                                if "hbm_stream_45MB_GBs" in ceilings else {}),
                             "single_buffer_cache_resident_us": round(us1, 2)}
            if not args.no_cpu:
                cms = cpu_median_ms(lambda: O2.int8_gemm(xq2c, wq2, sx2c, sw2c, fast=True), trials=5)
                cpu_c2[f"M{m}"] = {"ms": round(cms, 2), "GB/s": round(nbytes / (cms * 1e-3) / 1e9, 1)}
        extra["int8_gemv_11008x4096_hbm_ring"] = {"data": "BASELINE config 2 (seed 2)", **gemv}
        if cpu_c2:
            cpu_more["config2_int8_gemv"] = {
                "unit": "GB/s of the same algorithmic bytes", "cores": _cpu_threads(), "kind": "port",
                "sample": "the whole call at each M (exact int8 x int8 -> int32 matmul + scale epilogue -> bf16), "
                          "median of 5 after 1 warm-up", **cpu_c2}
        del ring

        # ---- the same shape with fp8 e4m3fn operands and per-tensor steps (seed-2 tensors, the
        # oracle's quantizer): the row-range decode kernel on the fp8 MFMA, same weight ring
        sw8 = O2.dynamic_scale(w2).reshape(1)
        w8c, _ = O2.fp8_quantize(w2, sw8, 0)
        ring8 = [w8c.to(dev).clone() for _ in range(10)]
        sw8d = sw8.to(dev)
        gemv8 = {}
        for m in (1, 4, 16, 64):
            sx8 = O2.dynamic_scale(x2_all[:m]).reshape(1)
            x8c, _ = O2.fp8_quantize(x2_all[:m], sx8, 0)
            x8, sx8d = x8c.to(dev), sx8.to(dev)
            y8 = torch.empty(m, N2, device=dev, dtype=torch.bfloat16)

            def launch8(i, x8=x8, sx8d=sx8d, y8=y8, m=m):
                check(lib.astrai_w8a8_gemm_fp8_pt(
                    x8.data_ptr(), ring8[i % len(ring8)].data_ptr(), sx8d.data_ptr(), sw8d.data_ptr(), None,
                    None, y8.data_ptr(), m, N2, K2, 0, 0, torch.cuda.current_stream().cuda_stream))

            us = _graph_us(launch8)
            nbytes = N2 * K2 + m * K2 + 2 * m * N2 + 8
            gbs = nbytes / (us * 1e-6) / 1e9
            gemv8[f"M{m}"] = {"us": round(us, 2), "GB/s": round(gbs, 0),
                              "frac_hbm_peak": round(gbs / PEAK_HBM_GBS, 4)}
        extra["fp8_gemv_11008x4096_hbm_ring"] = {"data": "BASELINE config 2 tensors (seed 2) as e4m3fn, per-tensor steps",
                                                 **gemv8}
        del ring8

        # ---- config 0: 16 x 2048 x 2048 int8 linear (launch-latency bound), seed-0 tensors
        xc, wc, _ = O2.make_inputs(0, 16, 2048, 2048)
        wq0c, sw0c = O2.int8_quantize_rows(wc)
        xq0c, sx0c = O2.int8_quantize_rows(xc)
        x0, w0 = xq0c.to(dev), wq0c.to(dev)
        s0, s1 = sx0c.reshape(-1).to(dev), sw0c.reshape(-1).to(dev)
        y0 = torch.empty(16, 2048, device=dev, dtype=torch.bfloat16)

        def launch0(i):
            check(lib.astrai_w8a8_gemm_int8_ptpc(x0.data_ptr(), w0.data_ptr(), s0.data_ptr(),
                                                 s1.data_ptr(), None, y0.data_ptr(), 16, 2048, 2048,
                                                 0, torch.cuda.current_stream().cuda_stream))

        extra["int8_config0_16x2048x2048"] = {"data": "BASELINE config 0 (seed 0)",
                                              "us": round(_graph_us(launch0), 2)}
        if not args.no_cpu:
            cms = cpu_median_ms(lambda: O2.int8_linear(xc, wq0c, sw0c, fast=True), trials=5)
            extra["int8_config0_16x2048x2048"]["cpu_oracle_ms"] = round(cms, 3)
            cpu_more["config0_int8_linear"] = {
                "value": round(cms, 3), "unit": "ms", "cores": _cpu_threads(), "kind": "port",
                "sample": "the whole config-0 linear (per-token quantize, int32 matmul, scale -> bf16), "
                          "median of 5 after 1 warm-up"}

    if not args.no_extra and not args.no_model:
        extra["decoder_config4_int8"] = _bench_decoder(dev)
        if not args.no_cpu:
            cpu_more["config4_decoder"] = _cpu_decoder_baseline()
    if cpu_more:
        extra["cpu_baselines"] = cpu_more

    line = {
        "metric": "W8A8 GEMM TFLOPS/TOPS + % MFMA peak; decode GEMV GB/s + % HBM peak (1 GPU)",
        "value": round(value, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn", "data": "synthetic",
        "config": {"workload": "BASELINE config 1: fp8 e4m3fn per-tensor GEMM, M=N=K=4096, "
                               "fp32 accumulate, bf16 out, seed 1"},
        "roofline": roofline, "cpu_baseline": cpu_baseline, "extra": extra,
        "host": {**_host_info(), "cpu_threads_used": _cpu_threads(), "torch": torch.__version__},
        "measured_ceilings": ceilings,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
