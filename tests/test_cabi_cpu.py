"""CPU-side checks of the C ABI: the built library loads, exports every function the header
declares (no compute is called here), and the Python binding types all of them."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "qlinear.h")


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(ql_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("ql_quant_per_row", "ql_quant_per_tensor", "ql_quant_per_group", "ql_fake_quant",
                 "ql_gemm_w8a16", "ql_gemm_w8a8", "ql_gemm_workspace_bytes", "ql_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from nanovllm import _qlinear as Q
    assert os.path.exists(Q.LIB_PATH), "build libqlinear.so first: python nano-vllm-hw3_amd/build.py"
    lib = ctypes.CDLL(Q.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in qlinear.h but not exported"


def test_binding_covers_header():
    from nanovllm import _qlinear as Q
    assert sorted(Q.SIGNATURES) == declared_functions()
    lib = Q.load()
    assert lib.ql_version() >= 1


def test_argument_validation_needs_no_gpu():
    """Rejections happen before any HIP call, so they can be exercised on a CPU-only host."""
    from nanovllm import _qlinear as Q
    lib = Q.load()
    one = ctypes.c_void_p(16)   # never dereferenced: the calls below are rejected first
    assert lib.ql_gemm_w8a16(7, 0, one, one, one, None, one, 4, 64, 128, 0, None, 0, None) == -1
    assert b"bad argument" in lib.ql_last_error()
    assert lib.ql_gemm_w8a16(0, 0, one, one, one, None, one, 4, 64, 100, 0, None, 0, None) == -2
    assert b"multiple of 32" in lib.ql_last_error()
    assert lib.ql_gemm_w8a16(0, 2, one, one, one, None, one, 4, 64, 256, 96, None, 0, None) == -2    # K % group
    assert lib.ql_gemm_w8a16(0, 2, one, one, one, None, one, 4, 64, 240, 48, None, 0, None) == -2    # K % 32
    # (a group size that is not a multiple of 32 is valid for the plain GEMM; its fused forms do not exist)
    assert lib.ql_gemm_w8a16_silu(0, 2, one, one, one, None, one, 4, 64, 192, 48, None, 0, None) == -2
    assert b"multiple of 32" in lib.ql_last_error()
    assert lib.ql_gemm_w8a16(0, 2, one, one, one, None, one, 4, 64, 192, 0, None, 0, None) == -2     # group <= 0
    assert lib.ql_quant_per_group(0, one, 4, 256, 96, one, one, None) == -2
    assert lib.ql_quant_per_row(0, one, 4, 100, one, one, None) == -2
    assert lib.ql_gemm_w8a8(0, one, one, one, None, None, one, 4, 64, 128, None, 0, None) == -1
    assert lib.ql_gemm_force_config(3, 4, 1, 4, 0) == -1
    assert lib.ql_gemm_force_config(0, 0, 0, 0, 0) == 0
    # workspace sizing is pure host arithmetic: 64 KiB of counters + split x tile slabs, or nothing
    assert lib.ql_gemm_force_config(1, 1, 4, 2, 4) == 0
    assert lib.ql_gemm_workspace_bytes(16, 64, 2048, 0) == 65536 + 2 * 4 * (1 * 1 * 16 * 64 * 4)
    assert lib.ql_gemm_force_config(0, 0, 0, 0, 0) == 0
    assert lib.ql_gemm_workspace_bytes(4096, 4096, 1024, 0) == 0


def test_workspace_max_covers_every_row_count():
    """ql_gemm_workspace_max_bytes(max_M) is the maximum of ql_gemm_workspace_bytes over 1..max_M (brute force), so
    one reservation covers decode buckets and eager prefill batches alike; includes the Qwen3-4B down_proj shape
    whose M = 600 call needs more than any M <= 512."""
    from nanovllm import _qlinear as Q
    lib = Q.load()
    for (N, K) in [(1024, 3072), (2560, 9728), (2048, 6144), (4096, 1024), (64, 256)]:
        for gran in (0, 2):
            brute = max(lib.ql_gemm_workspace_bytes(m, N, K, gran) for m in range(1, 2101))
            assert lib.ql_gemm_workspace_max_bytes(2100, N, K, gran) == brute
    assert lib.ql_gemm_workspace_max_bytes(16384, 2560, 9728, 0) >= lib.ql_gemm_workspace_bytes(600, 2560, 9728, 0)
    # (the built-in heuristics alone: measured plans of the shipped table may split the decode sizes further)
    lib.ql_gemm_plan_clear()
    try:
        assert lib.ql_gemm_workspace_max_bytes(16384, 2560, 9728, 0) >= lib.ql_gemm_workspace_bytes(600, 2560, 9728, 0) > \
            lib.ql_gemm_workspace_max_bytes(512, 2560, 9728, 0)
    finally:
        Q.load_plan_table(Q.PLAN_TABLE)
    assert lib.ql_gemm_workspace_max_bytes(0, 64, 256, 0) == 0


def test_ops_refuse_cpu_tensors():
    """No silent CPU fallback: the operator layer raises on non-GPU tensors."""
    import torch
    from nanovllm import _qlinear as Q
    from nanovllm.utils import quantization as NQ
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(Q.QLinearError):
        NQ.per_row_quant(x, torch.int8)
    with pytest.raises(Q.QLinearError):
        NQ.per_group_quant(x, 64, torch.int8)


# ---- libseqmix (include/seqmix.h) --------------------------------------------------------------------------------------
SEQMIX_HEADER = os.path.join(ROOT, "include", "seqmix.h")


def seqmix_declared():
    src = re.sub(r"/\*.*?\*/", "", open(SEQMIX_HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(sm_[a-z0-9_]+)\s*\(", src)))


def test_seqmix_binding_covers_header_and_library_exports_it():
    from nanovllm import _seqmix as SM
    SM.build_if_missing()
    lib = ctypes.CDLL(SM.LIB_PATH)
    names = seqmix_declared()
    assert sorted(SM.SIGNATURES) == names
    for name in names:
        assert hasattr(lib, name), f"{name} declared in seqmix.h but not exported"
    assert SM.load().sm_version() >= 1


def test_seqmix_argument_validation_needs_no_gpu():
    from nanovllm import _seqmix as SM
    lib = SM.load()
    one = ctypes.c_void_p(16)   # never dereferenced: the calls below are rejected first
    assert lib.sm_stream_step(7, one, one, one, one, one, one, 1e-5, one, 4, 2, 64, None) == -1          # unknown dtype
    assert lib.sm_stream_step(1, one, one, one, one, one, one, 1e-5, one, 4, 9, 64, None) == -2          # too many streams
    assert b"streams" in lib.sm_last_error()
    assert lib.sm_canon_conv(1, one, one, one, 3, 3, one, one, one, one, one, 4, 64, 4, None) == -1      # run >= runs
    assert lib.sm_latent_attn_tiles(one, one, one, one, one, one, 0.1, 2, 8, 4, 36, 64, 4, 0, 0, None) == -2   # R % 8
    assert lib.sm_latent_attn_tiles(one, one, one, one, one, one, 0.1, 2, 8, 4, 64, 48, 4, 0, 0, None) == -2   # block % 64
    assert lib.sm_latent_attn_tiles(one, one, one, one, one, one, 0.1, 2, 8, 4, 64, 64, 4, 72, 0, None) == -1   # values wider than the row
    assert lib.sm_latent_rope_store(1, one, 40, one, 1e-5, one, 96, one, one, 12, one, one, one, 4, 2, 16, 32, 8, None) == -1   # rotation wider than the part
    assert lib.sm_latent_attn_decode(one, one, one, one, one, 0.1, 2, 4, 64, 64, 4, 2, one, 16, 0, 0, None) == -3   # workspace
    assert lib.sm_moe_route(1, one, one, one, one, 4, 64, 8, 3, 4, 1, 0, None, 1, 1, None, None) == -2    # top > keep * E/groups
    assert lib.sm_moe_route(1, one, one, one, one, 4, 64, 8, 2, 4, 2, 5, None, 1, 1, None, None) == -1    # unknown score function
    assert lib.sm_moe_grouped(one, one, one, one, one, None, 1.0, 1.7, 0, one, 4, 2, 8, 60, 64, one, one, one, one, one, None) == -2
    assert lib.sm_moe_grouped(one, one, one, one, one, None, 1.0, 1.7, 9, one, 4, 2, 8, 64, 64, one, one, one, one, one, None) == -1   # unknown activation


# ---- libhymix (include/hymix.h) ----------------------------------------------------------------------------------------
HYMIX_HEADER = os.path.join(ROOT, "include", "hymix.h")


def hymix_declared():
    src = re.sub(r"/\*.*?\*/", "", open(HYMIX_HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(hm_[a-z0-9_]+)\s*\(", src)))


def test_hymix_binding_covers_header_and_library_exports_it():
    from nanovllm import _hymix as HM
    HM.build_if_missing()
    lib = ctypes.CDLL(HM.LIB_PATH)
    names = hymix_declared()
    assert sorted(HM.SIGNATURES) == names
    for name in names:
        assert hasattr(lib, name), f"{name} declared in hymix.h but not exported"
    assert HM.load().hm_version() >= 1


def test_hymix_argument_validation_needs_no_gpu():
    from nanovllm import _hymix as HM
    lib = HM.load()
    one = ctypes.c_void_p(16)   # never dereferenced: the calls below are rejected first
    assert lib.hm_embed_scaled(7, one, one, 1.0, one, 4, 64, None) == -1                                  # unknown dtype
    assert lib.hm_sublayer_close(1, one, one, None, 64, one, one, 0.5, None, 1e-5, None, None, None, 0, None, None, None, 4,
                                 64, None) == -1                                                          # a result without its gate
    assert lib.hm_sublayer_close(1, one, None, None, 0, None, None, 0.5, one, 1e-5, one, None, None, 0, None, None, None, 4,
                                 1 << 20, None) == -2                                                     # wider than the row buffer
    assert lib.hm_qkv_prepare(1, one, 100, 4, 3, 16, 8, None, None, 1e-5, one, 4, 0, one, one, one, one, None, 0, None, one, 4,
                              None, None, None, 0, 1.0, 0, None) == -1                                    # heads % kv_heads
    assert lib.hm_qkv_prepare(1, one, 200, 4, 2, 16, 8, None, None, 1e-5, one, 9, 0, one, one, one, one, None, 0, None, one, 4,
                              None, None, None, 1, 1.0, 0, None) == -1                                    # rotation wider than a head
    assert lib.hm_attn_tiles(one, one, one, one, one, one, None, 0, 0, 0.1, one, 2, 8, 4, 2, 20, 16, 64, 4, None, None, 0, 0, 0, None, 0, None) == -2   # dim % 8
    assert lib.hm_attn_tiles(one, one, one, one, one, one, None, 0, 0, 0.1, one, 2, 8, 4, 2, 16, 16, 48, 4, None, None, 0, 0, 0, None, 0, None) == -2   # block % 64
    assert lib.hm_attn_tiles(one, one, one, one, one, one, None, 0, 0, 0.1, one, 2, 8, 4, 2, 16, 16, 64, 4, one, one, 12, 6, 0, None, 0, None) == -1   # pooled blocks without a window
    assert lib.hm_attn_rows(1, one, one, one, one, one, one, None, 40, 0, 0.1, one, 4, 4, 2, 16, 16, 64, 4, one, one, 12, 5, 0, None, 0, None) == -1   # pooled pages too small
    assert lib.hm_group_norm_residual(1, one, one, None, one, None, 3, 1e-5, None, 4, 64, None) == -1     # groups do not divide the width
    assert lib.hm_attn_decode(one, one, one, one, one, None, 0, 0, 0.1, one, 2, 4, 2, 64, 64, 64, 4, 2, one, 16, None, None, 0, 0, 0, None, 0, None) == -3  # workspace
    assert b"workspace" in lib.hm_last_error()
    assert lib.hm_attn_rows(1, one, one, one, one, one, one, None, 0, 0, 0.1, one, 4, 4, 2, 16, 16, 64, 4, None, None, 0, 0, 8, one, 0,
                            None) == -1                                                                   # a head bias without sigmoid weights
    assert lib.hm_attn_tiles(one, one, one, one, one, one, one, 0, 0, 0.1, one, 2, 8, 4, 2, 16, 16, 64, 4, None, None, 0, 0, 8, None, 1,
                             None) == -1                                                                  # sigmoid weights with a sink
    assert lib.hm_attn_rows(1, one, one, one, one, one, one, None, 9, 2, 0.1, one, 4, 4, 2, 16, 16, 64, 4, None, None, 0, 0, 8, None, 0,
                            None) == -1                                                                   # a chunked mask with kept first tokens
    assert lib.hm_lightning_recurrence(1, one, 40, 0, 16, 32, one, one, one, one, one, one, 2, 2, 8, 8, 1, None) == -1   # rows narrower than the columns
    assert lib.hm_lightning_recurrence(1, one, 4096, 0, 1024, 2048, one, one, one, one, one, one, 2, 2, 512, 8, 1, None) == -2   # dim > 256
    assert lib.hm_dyt_residual(1, one, one, None, one, None, one, None, None, None, None, 4, 64, None) == -1   # a norm without its bias
    assert lib.hm_delta_recurrence(1, one, one, 10, one, one, one, one, one, 2, 2, 8, 1, None) == -1     # v rows narrower than heads * dim
    assert lib.hm_delta_recurrence(1, one, one, 1024, one, one, one, one, one, 2, 2, 512, 1, None) == -2  # dim > 256
