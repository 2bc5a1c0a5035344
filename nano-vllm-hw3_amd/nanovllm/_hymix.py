"""ctypes binding of libhymix.so (the C ABI declared in include/hymix.h): scaled embedding, the gated sublayer boundary
with norms on both sides, token shift with carried state, rotary attention over a paged key/value cache with sinks and
windows, chunked masks and sigmoid weights, the generalized delta rule and linear attention with a constant decay with their
per-sequence states, squared ReLU, the grouped-norm and tanh-norm residual boundaries.  No fallback on a GPU: a missing library
raises (``build_if_missing`` compiles it in-tree first, which needs hipcc but no GPU)."""
import ctypes
import os

import torch

from nanovllm._qlinear import QLinearError, _Workspace, require_cuda, stream_ptr  # noqa: F401  (shared helpers)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("HYMIX_LIB") or os.path.join(_HERE, "_lib", "libhymix.so")

HM_F32, HM_BF16 = 0, 1
_vp, _i64, _int, _sz, _f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float

# name -> (restype, argtypes); must list every function of include/hymix.h
SIGNATURES = {
    "hm_version": (_int, []),
    "hm_last_error": (ctypes.c_char_p, []),
    "hm_embed_scaled": (_int, [_int, _vp, _vp, _f, _vp, _i64, _int, _vp]),
    "hm_sublayer_close": (_int, [_int, _vp, _vp, _vp, _i64, _vp, _vp, _f, _vp, _f, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _i64,
                                 _int, _vp]),
    "hm_token_shift": (_int, [_int, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp]),
    "hm_qkv_prepare": (_int, [_int, _vp, _i64, _int, _int, _int, _int, _vp, _vp, _f, _vp, _int, _int, _vp, _vp, _vp, _vp, _vp,
                              _i64, _vp, _vp, _i64, _vp, _vp, _vp, _int, _f, _int, _vp]),
    "hm_attn_rows": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _f, _vp, _i64, _int, _int, _int, _int, _int,
                            _int, _vp, _vp, _int, _int, _int, _vp, _int, _vp]),
    "hm_pool_blocks": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _int, _int, _int, _int, _int, _vp]),
    "hm_attn_tiles": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _f, _vp, _int, _int, _int, _int, _int, _int, _int, _int,
                             _vp, _vp, _int, _int, _int, _vp, _int, _vp]),
    "hm_attn_decode_workspace_bytes": (_sz, [_i64, _int, _int, _int]),
    "hm_attn_decode": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _f, _vp, _i64, _int, _int, _int, _int, _int, _int, _int,
                              _vp, _sz, _vp, _vp, _int, _int, _int, _vp, _int, _vp]),
    "hm_lightning_recurrence": (_int, [_int, _vp, _i64, _int, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int,
                                       _int, _vp]),
    "hm_dyt_residual": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _vp]),
    "hm_group_norm_residual": (_int, [_int, _vp, _vp, _vp, _vp, _vp, _int, _f, _vp, _i64, _int, _vp]),
    "hm_scale_softcap": (_int, [_vp, _i64, _f, _f, _vp]),
    "hm_delta_prepare": (_int, [_int, _vp, _i64, _int, _int, _int, _int, _vp, _vp, _vp, _int, _f, _f, _vp, _i64, _int, _int, _vp]),
    "hm_delta_recurrence": (_int, [_int, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _int, _vp]),
    "hm_delta_gate_norm": (_int, [_int, _vp, _vp, _i64, _vp, _f, _vp, _i64, _int, _int, _vp]),
    "hm_relu_squared": (_int, [_int, _vp, _i64, _vp, _i64, _int, _vp]),
}

_lib = None


def build_if_missing():
    """Compile libhymix.so in-tree when it is not there (a fresh checkout); only this library, not the package's others."""
    if os.path.exists(LIB_PATH):
        return
    import importlib.util
    spec = importlib.util.spec_from_file_location("nanovllm_build", os.path.join(os.path.dirname(_HERE), "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.build(verbose=False, target="hymix")


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QLinearError(f"{LIB_PATH} not found: build it with `python nano-vllm-hw3_amd/build.py hymix`; "
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
        raise QLinearError(f"libhymix error {rc}: {load().hm_last_error().decode()}")


def dtype_code(dtype):
    if dtype == torch.float32:
        return HM_F32
    if dtype == torch.bfloat16:
        return HM_BF16
    raise QLinearError(f"storage type must be float32 or bfloat16, got {dtype}")


def ptr(t):
    return t.data_ptr() if t is not None else None


decode_workspace = _Workspace()     # partial states of split-key decode attention
