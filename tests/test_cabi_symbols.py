"""The C-ABI library loads and exports every function include/astrai_w8a8.h declares
(no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

from astrai_amd.extension import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "astrai_w8a8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(astrai_w8a8_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    assert names == sorted(_cabi.PROTOTYPES), (names, sorted(_cabi.PROTOTYPES))


def test_library_loads_and_exports_every_declared_symbol():
    assert os.path.exists(_cabi.LIB_PATH), "build with `make -C astrai_amd/csrc`"
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name
    lib.astrai_w8a8_abi_version.restype = ctypes.c_int
    assert lib.astrai_w8a8_abi_version() == _cabi.ABI_VERSION
    lib.astrai_w8a8_last_error.restype = ctypes.c_char_p
    assert lib.astrai_w8a8_last_error() == b""


def test_argument_validation_needs_no_gpu():
    lib = _cabi.load()
    assert lib is not None, _cabi.load_error()
    # null pointers are rejected before anything touches the device
    rc = lib.astrai_w8a8_gemm_int8_ptpc(None, None, None, None, None, None, 4, 4, 64, 0, None)
    assert rc == 1
    assert b"null" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_quantize_bf16_fp8(16, 16, 16, None, 8, 7, None)
    assert rc == 1 and b"fmt" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemv_int8_ptpc(16, 16, 16, 16, None, 16, 129, 4, 256, 0, None)
    assert rc == 2 and b"M <= 128" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_block128(16, 16, 16, 16, None, 16, 4, 4, 100, None)
    assert rc == 2 and b"128" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_pt(16, 16, 16, 16, None, None, 16, 4, 4, 64, 0, 1, None)
    assert rc == 1 and b"out_scale" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_pt(8, 16, 16, 16, None, None, 16, 4, 4, 64, 0, 0, None)
    assert rc == 1 and b"aligned" in lib.astrai_w8a8_last_error()
    # the per-workgroup-maxima forms of the quantizer, the amax pass and the ring push
    rc = lib.astrai_w8a8_quantize_bf16_fp8_partials(16, 16, 16, None, 64, 0, None)
    assert rc == 1 and b"null" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_quantize_bf16_fp8_partials(16, 16, 16, 16, 0, 0, None)
    assert rc == 1 and b"positive" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_quantize_bf16_fp8_partials(16, 24, 16, 16, 64, 0, None)
    assert rc == 1 and b"aligned" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_amax_bf16_partials(16, None, 64, None)
    assert rc == 1 and b"null" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_amax_ring_push_partials(16, 4, 4, 16, None, 16, 448.0, 1.0, None)
    assert rc == 1 and b"idx" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_amax_ring_push_partials(16, 4, 0, 16, None, 16, 0.0, 1.0, None)
    assert rc == 1 and b"positive" in lib.astrai_w8a8_last_error()
    assert _cabi.AMAX_PARTIALS == int(re.search(r"#define ASTRAI_W8A8_AMAX_PARTIALS\s+(\d+)", open(
        os.path.join(ROOT, "include", "astrai_w8a8.h")).read()).group(1))
    assert isinstance(lib.astrai_w8a8_last_kernel(), bytes)
    # the residual entry: residual required, aligned, and apart from the output
    rc = lib.astrai_w8a8_gemm_int8_ptpc_resid(16, 16, 16, 16, None, None, 4096, 4, 4, 64, None)
    assert rc == 1 and b"residual" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_int8_ptpc_resid(16, 16, 16, 16, None, 4100, 8192, 4, 4, 64, None)
    assert rc == 1 and b"aligned" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_int8_ptpc_resid(16, 16, 16, 16, None, 4096, 4112, 4, 4, 64, None)
    assert rc == 1 and b"overlaps" in lib.astrai_w8a8_last_error()


def test_shape_predicates_agree_with_the_entry_points():
    """Just past each limit the Python predicate says no and the entry point returns
    UNSUPPORTED (status 2) before anything touches the device; 16 stands for an
    aligned non-null pointer that is never dereferenced."""
    lib = _cabi.load()
    assert lib is not None, _cabi.load_error()
    P = 16

    def decode(n_heads, n_kv, seq, hd):
        return lib.astrai_w8a8_attn_decode_bf16(P, P, P, P, P, 1 << 30, P, None, None, 1, seq, n_heads, n_kv,
                                                hd, 64, 1, 1.0, None)

    for shape in ((128, 16, 1, 128), (16, 4, 3, 128), (16, 4, 1, 64)):   # > 64 heads, > 8 rows, head_dim
        assert not _cabi.attn_decode_supported(*shape), shape
        assert decode(*shape) == 2, (shape, lib.astrai_w8a8_last_error())
    assert _cabi.attn_decode_supported(64, 8, 1, 128) and _cabi.attn_decode_supported(16, 4, 2, 128)

    def prefill(n_heads, n_kv, hd):
        return lib.astrai_w8a8_attn_prefill_bf16(P, P, P, P, P, 1, 8, n_heads, n_kv, hd, 64, 1.0, None)

    for shape in ((16, 16, 128), (48, 3, 128), (16, 4, 64)):
        assert not _cabi.attn_prefill_supported(*shape), shape
        assert prefill(*shape) == 2, (shape, lib.astrai_w8a8_last_error())

    def rope_gemm(tokens, k, hd, n_heads, n_kv):
        return lib.astrai_w8a8_gemm_int8_ptpc_rope_cache(P, P, P, P, P, P, P, P, P, tokens, 1, n_heads, n_kv,
                                                         hd, 64, k, None)

    for tokens, k, hd, n_heads, n_kv in ((65, 256, 128, 4, 1), (8, 128, 128, 4, 1), (8, 256, 6, 4, 1),
                                         (8, 1 << 16, 128, 200, 28)):        # last: 2 GiB weight
        n = (n_heads + 2 * n_kv) * hd
        assert not _cabi.mm_int8_rope_cache_supported(tokens, k, hd, n), (tokens, k, hd, n)
        assert rope_gemm(tokens, k, hd, n_heads, n_kv) == 2, lib.astrai_w8a8_last_error()
    assert _cabi.mm_int8_rope_cache_supported(64, 2048, 128, 3072)

    for width in (8200, 12, 11008):
        assert not _cabi.fused_rows_supported(width)
        assert lib.astrai_w8a8_add_rmsnorm_quantize_int8_rows(P, None, P, 1e-5, None, None, P, P, 4, width,
                                                              None) == 2
        assert lib.astrai_w8a8_silu_mul_quantize_int8_rows(P, P, max(width, 16) + (-width) % 8, None, P, P, 4,
                                                           width, None) == 2
    assert _cabi.fused_rows_supported(8192) and _cabi.fused_rows_supported(5632)
    header = open(os.path.join(ROOT, "astrai_amd", "csrc", "launchers.h")).read()
    assert int(re.search(r"kFusedRowMax\s*=\s*(\d+)", header).group(1)) == _cabi.FUSED_ROW_MAX


def test_fuse_int8_weights_refuses_widths_the_fused_producers_reject():
    import pytest
    import torch
    from astrai_amd.model import AutoRegressiveLM, AutoRegressiveLMConfig, fuse_int8_weights
    cfg = AutoRegressiveLMConfig(vocab_size=32, hidden_size=64, num_hidden_layers=1, num_attention_heads=2,
                                 num_key_value_heads=1, intermediate_size=8200, max_position_embeddings=8)
    with pytest.raises(ValueError, match="intermediate_size 8200"):
        fuse_int8_weights(AutoRegressiveLM(cfg).to(torch.bfloat16))


def test_decode_attention_split_plan():
    """Up to 512 workgroups, at most eight splits, none shorter than ~160 keys of the longest context."""
    assert _cabi.decode_nsplit(128, 640) == 4      # config 4: 32 sequences x 4 KV heads, 512 + 128 tokens
    assert _cabi.decode_nsplit(8, 640) == 4
    assert _cabi.decode_nsplit(256, 640) == 2
    assert _cabi.decode_nsplit(8, 2048) == 8
    assert _cabi.decode_nsplit(256, 4096) == 2 and _cabi.decode_nsplit(1024, 4096) == 1
    assert _cabi.decode_nsplit(1, 64) == 1
    assert _cabi.decode_nsplit(0, 0) == 1


def test_k_padding_plan_of_the_wrappers():
    """Which products the wrappers re-lay with zero codes (K % 16 != 0 and at least 2^24
    multiply-adds) and to which K; values and the zero tail, on CPU tensors."""
    import torch

    a = torch.randint(-127, 128, (300, 1032), dtype=torch.int8)
    b = torch.randint(-127, 128, (520, 1032), dtype=torch.int8)
    pa, pb, kp = _cabi._pad_k(a, b)
    assert kp == 1152 and pa.shape == (300, kp) and pb.shape == (520, kp) and pa.dtype == torch.int8
    assert torch.equal(pa[:, :1032], a) and not pa[:, 1032:].any() and not pb[:, 1032:].any()
    assert _cabi._pad_k(a[:64], b)[2] == 1280          # decode kernels take whole 256-byte items
    assert _cabi._pad_k(a[:, :1024].contiguous(), b[:, :1024].contiguous())[0].shape == (300, 1024)  # K % 16 == 0
    assert _cabi._pad_k(a[:8], b[:8])[2] == 1032        # too small to repay the copies
    f = torch.randn(300, 1032).to(torch.float8_e4m3fn)
    pf = _cabi._pad_k(f, b.view(torch.float8_e4m3fn))[0]
    assert pf.dtype == torch.float8_e4m3fn and torch.equal(pf[:, :1032].view(torch.uint8), f.view(torch.uint8))
    assert not pf[:, 1032:].view(torch.uint8).any()


def test_bench_refuses_more_than_one_gpu():
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "--gpus 1" in r.stderr and not r.stdout.strip()
