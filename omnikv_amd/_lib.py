"""ctypes binding of libomnikv_hip.so (declared in include/omnikv_hip.h).

The library is required: there is no CPU or torch fallback.  `lib()` raises
OmniKVLibraryError when the shared object has not been built, and every wrapper
turns a negative status into an exception carrying okv_last_error().
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libomnikv_hip.so")
DIAG_LIB_PATH = os.path.join(_PKG, "libomnikv_hip_diag.so")  # measurement build: + the okv_diag_* hooks
STAMPS_LIB_PATH = os.path.join(_PKG, "libomnikv_hip_stamps.so")  # timeline build (csrc/build.py --stamps): + device timestamps

OKV_F32, OKV_BF16, OKV_F16 = 0, 1, 2
OKV_REDUCE_MAX, OKV_REDUCE_SUM = 0, 1
OKV_NORM_RAW, OKV_NORM_SOFTMAX = 0, 1
OKV_OP_SCORE, OKV_OP_TOPK, OKV_OP_DENSE_ATTN, OKV_OP_SPARSE_ATTN, OKV_OP_SCORE_WINDOW = 0, 1, 2, 3, 4
OKV_OP_DENSE_ATTN_SELECT, OKV_OP_DENSE_ATTN_WINDOW = 5, 6

EXPORTS = (
    "okv_strerror",
    "okv_last_error",
    "okv_version",
    "okv_workspace_bytes",
    "okv_set_option",
    "okv_score",
    "okv_score_window",
    "okv_topk",
    "okv_dense_attn",
    "okv_dense_attn_select",
    "okv_dense_attn_window",
    "okv_sparse_attn",
    "okv_sparse_attn_noalloc",
    "okv_noalloc_scratch_bytes",
    "okv_gather_rows",
    "okv_offload_stage",
    "okv_offload_plan",
    "okv_offload_fetch",
    "okv_rmsnorm",
    "okv_rope",
    "okv_rope_append",
    "okv_silu_mul",
)


class OmniKVLibraryError(RuntimeError):
    pass


class KVLayout(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("num_q_heads", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("token_stride", C.c_int64),
        ("head_stride", C.c_int64),
        ("batch_stride", C.c_int64),
        ("page_table", C.c_void_p),
        ("page_size", C.c_int32),
        ("page_table_stride", C.c_int32),
        ("page_stride", C.c_int64),
    ]


class Shape(C.Structure):
    _fields_ = [
        ("batch", C.c_int32),
        ("num_q_heads", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("head_dim", C.c_int32),
        ("max_seq_len", C.c_int32),
        ("max_tail_len", C.c_int32),
        ("with_scores", C.c_int32),
    ]


_lib = None


def _declare(l):
    vp, i32, i64, f32, sz = C.c_void_p, C.c_int32, C.c_int64, C.c_float, C.c_size_t
    l.okv_strerror.restype = C.c_char_p
    l.okv_strerror.argtypes = [C.c_int]
    l.okv_last_error.restype = C.c_char_p
    l.okv_last_error.argtypes = []
    l.okv_version.restype = C.c_int
    l.okv_version.argtypes = []
    l.okv_workspace_bytes.restype = C.c_int
    l.okv_workspace_bytes.argtypes = [C.c_int, C.POINTER(Shape), C.POINTER(sz)]
    l.okv_set_option.restype = C.c_int
    l.okv_set_option.argtypes = [C.c_char_p, C.c_int]
    if hasattr(l, "okv_diag_split_pass_only"):  # the measurement build only; not part of the public header
        l.okv_diag_split_pass_only.restype = C.c_int
        l.okv_diag_split_pass_only.argtypes = [C.c_int]
        l.okv_diag_split_geometry.restype = C.c_int
        l.okv_diag_split_geometry.argtypes = [C.c_int, C.POINTER(Shape), C.POINTER(i32), C.POINTER(i32)]
        l.okv_diag_gather_floor.restype = C.c_int
        l.okv_diag_gather_floor.argtypes = [vp, vp, C.POINTER(KVLayout), vp, i64, vp, i32, i32, i32, i32, vp, vp]
        l.okv_diag_empty_launch.restype = C.c_int
        l.okv_diag_empty_launch.argtypes = [vp, vp]
    if hasattr(l, "okv_stamps_read"):  # the timeline build only
        l.okv_stamps_read.restype = C.c_int
        l.okv_stamps_read.argtypes = [C.c_int, vp, C.c_int]
    l.okv_score.restype = C.c_int
    l.okv_score.argtypes = [vp, vp, C.POINTER(KVLayout), vp, i32, i32, i32, i32, f32, vp, i64, vp, sz, vp]
    l.okv_score_window.restype = C.c_int
    l.okv_score_window.argtypes = [vp, i64, i64, i64, i32, i32, vp, C.POINTER(KVLayout), vp, i32, i32, f32, vp, i64,
                                   vp, sz, vp]
    l.okv_topk.restype = C.c_int
    l.okv_topk.argtypes = [vp, i64, vp, i32, vp, i32, i32, vp, i64, vp, sz, vp]
    l.okv_dense_attn.restype = C.c_int
    l.okv_dense_attn.argtypes = [vp, vp, vp, C.POINTER(KVLayout), vp, i32, i32, f32, vp, vp, i32, i32, i32, vp, i64, vp, sz, vp]
    l.okv_dense_attn_select.restype = C.c_int
    l.okv_dense_attn_select.argtypes = l.okv_dense_attn.argtypes[:-3] + [vp, i32, vp, i64, vp, sz, vp]
    l.okv_dense_attn_window.restype = C.c_int
    l.okv_dense_attn_window.argtypes = [vp, vp, i64, i64, i64, i32, i32, vp, vp, C.POINTER(KVLayout), vp, i32, i32, f32,
                                        vp, vp, i32, vp, i64, vp, sz, vp]
    l.okv_sparse_attn.restype = C.c_int
    l.okv_sparse_attn.argtypes = [vp, vp, vp, C.POINTER(KVLayout), vp, i64, vp, i32, vp, vp, i64, i64, i64, vp, i32, i32, f32, vp, vp, sz, vp]
    l.okv_sparse_attn_noalloc.restype = C.c_int
    l.okv_sparse_attn_noalloc.argtypes = l.okv_sparse_attn.argtypes[:-3] + [vp]
    l.okv_noalloc_scratch_bytes.restype = C.c_int64
    l.okv_noalloc_scratch_bytes.argtypes = []
    l.okv_gather_rows.restype = C.c_int
    l.okv_gather_rows.argtypes = [vp, C.POINTER(KVLayout), vp, i64, vp, i32, i32, vp, i64, i64, i64, vp]
    l.okv_offload_plan.restype = C.c_int
    l.okv_offload_plan.argtypes = [vp, i32, vp, vp, i32, vp, vp, vp, vp]
    l.okv_offload_fetch.restype = C.c_int
    l.okv_offload_fetch.argtypes = [vp, i64, vp, vp, vp, i32, vp, vp]
    l.okv_rmsnorm.restype = C.c_int
    l.okv_rmsnorm.argtypes = [vp, vp, vp, f32, i32, i32, i32, vp, vp, vp]
    l.okv_rope.restype = C.c_int
    l.okv_rope.argtypes = [vp, i64, vp, i64, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp]
    l.okv_rope_append.restype = C.c_int
    l.okv_rope_append.argtypes = [vp, i64, vp, i64, vp, i64, vp, vp, i32, i32, i32, i32, i32, vp, vp, vp, i64, i64, i64,
                                  vp, i64, vp]
    l.okv_silu_mul.restype = C.c_int
    l.okv_silu_mul.argtypes = [vp, vp, i64, i32, vp, vp]
    l.okv_offload_stage.restype = C.c_int
    l.okv_offload_stage.argtypes = [vp, i64, vp, i32, vp, i32, vp, vp, vp]


_want_diag = False


def use_diag_build(stamps: bool = False) -> None:
    """Benchmarks call this before anything else touches the library: the process then loads the
    measurement build (the product's sources + the okv_diag_* hooks) instead of the product library;
    stamps=True: the timeline build (measurement build + device timestamps in two kernels)."""
    global _want_diag
    if _lib is not None and not hasattr(_lib, "okv_diag_split_pass_only"):
        raise OmniKVLibraryError("the product library is already loaded: call use_diag_build() first")
    _want_diag = "stamps" if stamps else True


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        path = STAMPS_LIB_PATH if _want_diag == "stamps" else DIAG_LIB_PATH if _want_diag else LIB_PATH
        if not os.path.exists(path):
            raise OmniKVLibraryError(
                f"{path} is missing: build it with `python omnikv_amd/csrc/build.py` "
                "(hipcc, gfx950). There is no fallback path."
            )
        l = C.CDLL(path)
        _declare(l)
        _lib = l
    return _lib


def check(status: int) -> None:
    if status != 0:
        l = lib()
        raise OmniKVLibraryError(
            f"{l.okv_strerror(status).decode()} ({status}): {l.okv_last_error().decode()}"
        )
