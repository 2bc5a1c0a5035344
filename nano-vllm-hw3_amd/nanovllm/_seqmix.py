"""ctypes binding of libseqmix.so (the C ABI declared in include/seqmix.h): multi-stream residuals, short causal
convolutions, latent attention, PolyNorm / clamped GLU and expert routing.  As with libqlinear there is no fallback
on a GPU: a missing library raises (``build_if_missing`` compiles it in-tree first, which needs hipcc but no GPU)."""
import ctypes
import os

import torch

from nanovllm._qlinear import QLinearError, _Workspace, require_cuda, stream_ptr  # noqa: F401  (shared helpers)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SEQMIX_LIB") or os.path.join(_HERE, "_lib", "libseqmix.so")

SM_F32, SM_BF16 = 0, 1
_vp, _i64, _int, _sz, _f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float

# name -> (restype, argtypes); must list every function of include/seqmix.h
SIGNATURES = {
    "sm_version": (_int, []),
    "sm_last_error": (ctypes.c_char_p, []),
    "sm_embed_streams": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "sm_stream_step": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _i64, _int, _int, _vp]),
    "sm_canon_conv": (_int, [_int, _vp, _vp, _vp, _int, _int, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "sm_canon_update": (_int, [_int, _vp, _vp, _int, _int, _vp, _vp, _int, _int, _int, _vp]),
    "sm_latent_norm_store": (_int, [_int, _vp, _i64, _vp, _f, _vp, _vp, _i64, _int, _vp]),
    "sm_rms_norm_rows": (_int, [_int, _vp, _i64, _vp, _f, _vp, _i64, _int, _vp]),
    "sm_latent_attn_rows": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _f, _i64, _int, _int, _int, _int, _int, _int, _vp]),
    "sm_latent_rope_store": (_int, [_int, _vp, _i64, _vp, _f, _vp, _i64, _vp, _vp, _int, _vp, _vp, _vp, _i64, _int, _int, _int,
                                    _int, _vp]),
    "sm_latent_attn_tiles": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _int, _int, _int, _int, _int, _int, _int, _int, _vp]),
    "sm_latent_decode_workspace_bytes": (_sz, [_i64, _int, _int, _int]),
    "sm_latent_attn_decode": (_int, [_vp, _vp, _vp, _vp, _vp, _f, _i64, _int, _int, _int, _int, _int, _vp, _sz, _int, _int, _vp]),
    "sm_poly_norm": (_int, [_int, _vp, _vp, _f, _vp, _i64, _int, _vp]),
    "sm_clamped_glu": (_int, [_int, _vp, _f, _f, _vp, _i64, _int, _vp]),
    "sm_moe_route": (_int, [_int, _vp, _vp, _vp, _vp, _i64, _int, _int, _int, _int, _int, _int, _vp, _int, _int, _vp, _vp]),
    "sm_moe_pairs_gate_up": (_int, [_int, _vp, _vp, _vp, _f, _f, _int, _vp, _i64, _int, _int, _int, _vp]),
    "sm_moe_pairs_down": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _int, _vp]),
    "sm_moe_grouped_tiles": (_int, [_i64, _int, _int]),
    "sm_moe_tiles128_count": (_int, [_i64, _int, _int]),
    "sm_moe_tiles128": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _int, _vp, _i64, _int, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp]),
    "sm_moe_align": (_int, [_vp, _i64, _int, _int, _vp, _vp, _vp, _vp]),
    "sm_moe_combine": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _vp]),
    "sm_moe_grouped": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _f, _int, _vp, _i64, _int, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp]),
}

_lib = None


def build_if_missing():
    """Compile libseqmix.so in-tree when it is not there (a fresh checkout); only this library, not the package's others."""
    if os.path.exists(LIB_PATH):
        return
    import importlib.util
    spec = importlib.util.spec_from_file_location("nanovllm_build", os.path.join(os.path.dirname(_HERE), "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build(verbose=False, target="seqmix")


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QLinearError(f"{LIB_PATH} not found: build it with `python nano-vllm-hw3_amd/build.py seqmix`; "
                           "these operators have no fallback on a GPU")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        raise QLinearError(f"libseqmix error {rc}: {load().sm_last_error().decode()}")


def dtype_code(dtype):
    if dtype == torch.float32:
        return SM_F32
    if dtype == torch.bfloat16:
        return SM_BF16
    raise QLinearError(f"storage type must be float32 or bfloat16, got {dtype}")


def ptr(t):
    return t.data_ptr() if t is not None else None


decode_workspace = _Workspace()     # partial states of split-key decode attention
