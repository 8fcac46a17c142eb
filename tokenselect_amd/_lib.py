"""ctypes binding of ``libtokenselect_hip.so`` (declared in ``include/tokenselect.h``).

The library is the product: there is no Python or CPU fallback.  If it has not
been built, loading raises with the build command.  ``import torch`` happens
first so that the HIP runtime the library binds to is the one PyTorch-ROCm has
already loaded (same ``libamdhip64.so`` soname, hence shared streams and memory).
"""

import ctypes
import os

import torch  # noqa: F401  (loads libamdhip64 before our library resolves it)

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libtokenselect_hip.so")

TS_OK, TS_EINVAL, TS_ESHAPE, TS_EWORKSPACE, TS_EHIP = 0, -1, -2, -3, -4
TS_ROPE_NONE, TS_ROPE_LLAMA = 0, 1
TS_HEADMAP_MOD, TS_HEADMAP_DIV = 0, 1
TS_DTYPE_F32, TS_DTYPE_BF16 = 0, 1

_i32, _i64, _f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_float
_ptr, _size = ctypes.c_void_p, ctypes.c_size_t


class TsConfig(ctypes.Structure):
    _fields_ = [
        ("num_heads", _i32), ("num_kv_heads", _i32), ("head_dim", _i32), ("page_size", _i32),
        ("n_init", _i32), ("n_local", _i32), ("top_k", _i32), ("pool_kernel", _i32),
        ("head_map", _i32), ("rope_mode", _i32),
        ("rope_theta", _f32), ("rope_scale", _f32), ("sm_scale", _f32), ("logit_cap", _f32),
    ]


class TsBatch(ctypes.Structure):
    _fields_ = [
        ("batch", _i32), ("max_seq_len", _i32), ("seq_lens", _ptr), ("table", _ptr),
        ("table_stride", _i64), ("k_per_req", _ptr), ("fault", _ptr), ("host_seq_lens", _ptr),
        ("threshold_hint", _ptr), ("separate_kernels", _i32), ("rerun", _i32), ("wait_us", ctypes.c_uint32),
        ("absent_workgroups", _i32), ("workspace_clean", _i32),
    ]


class TsSelCache(ctypes.Structure):
    _fields_ = [
        ("q_cache", _ptr), ("topk_cache", _ptr), ("cache_len", _ptr), ("counters", _ptr),
        ("threshold", _f32),
    ]


class TsPagePool(ctypes.Structure):
    _fields_ = [("free_pages", _ptr), ("free_count", _ptr), ("ticket", _ptr)]


class TsNewKv(ctypes.Structure):
    _fields_ = [("k", _ptr), ("v", _ptr), ("out_cache_loc", _ptr), ("pages", ctypes.POINTER(TsPagePool)),
                ("max_tokens", _i32)]


_CFG, _BT, _SC = ctypes.POINTER(TsConfig), ctypes.POINTER(TsBatch), ctypes.POINTER(TsSelCache)
_PP = ctypes.POINTER(TsPagePool)
_KV = ctypes.POINTER(TsNewKv)

# name -> (restype, argtypes); mirrors include/tokenselect.h one to one.
SIGNATURES = {
    "ts_version": (_i32, []),
    "ts_last_error": (ctypes.c_char_p, []),
    "ts_check_config": (_i32, [_CFG]),
    "ts_rope_apply": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _ptr]),
    "ts_paged_matmul": (_i32, [_ptr, _ptr, _i64, _ptr, _ptr, _i32, _i64, _i32, _i32, _i32, _ptr]),
    "ts_score_partials_bytes": (_size, [_CFG, _i32, _i32]),
    "ts_score_stride": (_i64, [_i32]),
    "ts_score": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _size, _ptr]),
    "ts_vote": (_i32, [_CFG, _BT, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "ts_score_vote_supported": (_i32, [_CFG, _i32, _i32]),
    "ts_score_vote": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _size, _ptr]),
    "ts_topk_workspace_bytes": (_size, [_CFG, _i32, _i32]),
    "ts_topk_ragged": (_i32, [_CFG, _BT, _ptr, _i64, _ptr, _SC, _ptr, _ptr, _i64, _ptr, _ptr,
                              _size, _ptr]),
    "ts_select_supported": (_i32, [_CFG, _i32, _i32]),
    "ts_select_workspace_bytes": (_size, [_CFG, _i32, _i32]),
    "ts_select": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _SC, _ptr, _ptr, _i64, _ptr, _ptr, _i64,
                         _ptr, _size, _ptr]),
    "ts_select_cleared": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _SC, _ptr, _ptr, _i64, _ptr, _ptr, _i64,
                         _ptr, _size, _ptr]),
    "ts_select_cleared_bounded": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _SC, _ptr, _ptr, _i64, _ptr,
                                         _ptr, _i64, _ptr, _size, ctypes.c_uint64, _i32, _ptr]),
    "ts_select_clear": (_i32, [_CFG, _BT, _ptr, _size, _ptr]),
    "ts_selcache_step": (_i32, [_CFG, _BT, _ptr, _SC, _ptr, _ptr]),
    "ts_attn_workspace_bytes": (_size, [_CFG, _i32, _i32]),
    "ts_sparse_decode_attn": (_i32, [_CFG, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i32, _i32,
                                     _ptr, _ptr, _size, _ptr]),
    "ts_attn_static_scratch_bytes": (_size, []),
    "ts_sparse_decode_attn_static": (_i32, [_CFG, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i32, _i32,
                                            _ptr, _ptr]),
    "ts_kv_store": (_i32, [_CFG, _ptr, _ptr, _ptr, _PP, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i32, _i32,
                           _ptr]),
    "ts_qkv_store": (_i32, [_CFG, _ptr, _ptr, _ptr, _i32, _ptr, _PP, _ptr, _ptr, _ptr, _i64, _ptr, _i64,
                            _ptr, _i32, _i32, _ptr]),
    "ts_kv_store_chunk": (_i32, [_CFG, _ptr, _ptr, _ptr, _PP, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _i32,
                                 _ptr]),
    "ts_fingerprint": (_i32, [_CFG, _ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr]),
    "ts_prefill_attn_workspace_bytes": (_size, [_CFG, _i32]),
    "ts_sparse_prefill_attn": (_i32, [_CFG, _ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _i32, _ptr, _ptr,
                                      _size, _ptr]),
    "ts_prefill_chunk": (_i32, [_CFG, _BT, _ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _ptr,
                                _ptr, _i64, _ptr, _ptr, _size, _ptr]),
    "ts_prefill_step": (_i32, [_CFG, _BT, _KV, _ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _ptr,
                               _ptr, _i64, _ptr, _ptr, _size, _ptr]),
    "ts_set_fused_select": (_i32, [_i32]),
    "ts_decode_layer_selection": (_i32, [_CFG, _i32, _i32]),
    "ts_decode_layer_selection_of": (_i32, [_CFG, _BT]),
    "ts_decode_layer_workspace_bytes": (_size, [_CFG, _i32, _i32]),
    "ts_decode_layer_votes": (_i32, [_CFG, _BT, _ptr, _ptr, _ptr, _ptr, _i64, _SC, _ptr, _i64, _ptr,
                                     _size, _ptr]),
    "ts_decode_layer_attend": (_i32, [_CFG, _BT, _ptr, _ptr, _i64, _ptr, _ptr, _i64, _SC, _ptr, _ptr,
                                      _ptr, _i64, _ptr, _ptr, _size, _ptr]),
    "ts_decode_layer": (_i32, [_CFG, _BT, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _SC, _ptr, _ptr,
                               _ptr, _i64, _ptr, _ptr, _size, _ptr]),
    "ts_decode_step": (_i32, [_CFG, _BT, _KV, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _SC, _ptr, _ptr,
                              _ptr, _i64, _ptr, _ptr, _size, _ptr]),
}

_lib = None


class TokenSelectError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libtokenselect_hip error {code}: {message}")
        self.code = code
        self.message = message


def load() -> ctypes.CDLL:
    """Load the built library; never builds, never falls back."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m tokenselect_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != TS_OK:
        raise TokenSelectError(code, load().ts_last_error().decode("utf-8", "replace"))
