"""ctypes binding of libfa_rocm.so (the C ABI declared in include/fa_rocm.h).

PyTorch is used for device memory and the current stream only: tensors are handed
to the library as raw device pointers with element strides."""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "csrc", "libfa_rocm.so")

FA_BF16, FA_FP16, FA_INT8 = 0, 1, 2
ABI_VERSION = 2     # FA_ROCM_ABI_VERSION of include/fa_rocm.h this binding was written against

_i32, _i64, _f32, _vp, _sz = C.c_int32, C.c_int64, C.c_float, C.c_void_p, C.c_size_t


class KvcacheArgs(C.Structure):
    """Mirror of struct fa_kvcache_args (include/fa_rocm.h); field order is the ABI."""
    _fields_ = (
        [(n, _vp) for n in ("q", "out", "softmax_lse", "k_cache", "v_cache", "k_scale_cache", "v_scale_cache",
                            "k_new", "v_new", "rotary_cos", "rotary_sin", "cache_seqlens", "block_table",
                            "workspace")]
        + [("workspace_bytes", _sz)]
        + [(n, _i32) for n in ("batch", "seqlen_q", "nheads", "nheads_k", "headdim_qk", "headdim_v", "seqlen_new",
                               "num_blocks", "page_size", "max_blocks_per_seq", "rotary_dim", "seqlen_ro")]
        + [(n, _i64) for n in ("q_stride_b", "q_stride_s", "q_stride_h", "o_stride_b", "o_stride_s", "o_stride_h",
                               "k_stride_block", "k_stride_row", "k_stride_h", "v_stride_block", "v_stride_row",
                               "v_stride_h", "ks_stride_block", "ks_stride_row", "kn_stride_b", "kn_stride_s",
                               "kn_stride_h", "vn_stride_b", "vn_stride_s", "vn_stride_h", "bt_stride_b")]
        + [("io_dtype", _i32), ("kv_dtype", _i32), ("softmax_scale", _f32), ("softcap", _f32), ("causal", _i32),
           ("window_left", _i32), ("window_right", _i32), ("rotary_interleaved", _i32), ("num_splits", _i32)]
    )


class VarlenArgs(C.Structure):
    """Mirror of struct fa_varlen_args (include/fa_rocm.h)."""
    _fields_ = (
        [(n, _vp) for n in ("q", "k", "v", "out", "softmax_lse", "cu_seqlens_q", "cu_seqlens_k", "seqused_k",
                            "block_table")]
        + [(n, _i32) for n in ("batch", "total_q", "nheads", "nheads_k", "headdim", "max_seqlen_q", "max_seqlen_k",
                               "page_size", "max_blocks_per_seq", "num_blocks")]
        + [(n, _i64) for n in ("q_stride_t", "q_stride_h", "k_stride_t", "k_stride_h", "v_stride_t", "v_stride_h",
                               "k_stride_block", "v_stride_block", "o_stride_t", "o_stride_h", "bt_stride_b")]
        + [("io_dtype", _i32), ("softmax_scale", _f32), ("softcap", _f32), ("causal", _i32), ("window_left", _i32),
           ("window_right", _i32), ("num_splits", _i32), ("workspace", _vp), ("workspace_bytes", _sz)]
    )


class SplitPlan(C.Structure):
    """Mirror of struct fa_split_plan (include/fa_rocm.h)."""
    _fields_ = [("mode", _i32), ("nsplits", _i32), ("split_keys", _i32), ("num_wgs", _i32), ("num_workers", _i32),
                ("min_share", _i32), ("workspace_bytes", _sz)]


EXPORTS = {
    "fa_rocm_abi_version": (C.c_int, []),
    "fa_rocm_reload_env": (None, []),
    "fa_rocm_last_error": (C.c_char_p, []),
    "fa_rocm_sizeof_kvcache_args": (_sz, []),
    "fa_rocm_sizeof_varlen_args": (_sz, []),
    "fa_rocm_sizeof_split_plan": (_sz, []),
    "fa_rocm_num_cus": (C.c_int, []),
    "fa_rocm_plan_kvcache": (C.c_int, [C.POINTER(KvcacheArgs), C.c_int, C.POINTER(SplitPlan)]),
    "fa_rocm_kvcache_workspace_bytes": (_sz, [C.POINTER(KvcacheArgs), C.c_int]),
    "fa_rocm_kvcache_validate": (C.c_int, [C.POINTER(KvcacheArgs)]),
    "fa_rocm_varlen_validate": (C.c_int, [C.POINTER(VarlenArgs)]),
    "fa_rocm_fwd_kvcache": (C.c_int, [C.POINTER(KvcacheArgs), _vp]),
    "fa_rocm_fwd_kvcache_profiled": (C.c_int, [C.POINTER(KvcacheArgs), _vp, C.POINTER(_vp)]),
    "fa_rocm_varlen_fwd": (C.c_int, [C.POINTER(VarlenArgs), _vp]),
    "fa_rocm_varlen_num_splits": (C.c_int, [C.POINTER(VarlenArgs), C.c_int]),
    "fa_rocm_varlen_workspace_bytes": (_sz, [C.POINTER(VarlenArgs), C.c_int]),
    "fa_rocm_append_kv": (C.c_int, [C.POINTER(KvcacheArgs), _vp]),
    "fa_rocm_fwd_kvcache_static": (C.c_int, [C.POINTER(KvcacheArgs), _vp]),
}

_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Load the HIP library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python flash-attention-npu_amd/build.py` "
                "(flash_attn_npu has no CPU or PyTorch fallback)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        if lib.fa_rocm_abi_version() != ABI_VERSION:
            raise RuntimeError("libfa_rocm.so ABI version mismatch")
        if (lib.fa_rocm_sizeof_kvcache_args() != C.sizeof(KvcacheArgs)
                or lib.fa_rocm_sizeof_varlen_args() != C.sizeof(VarlenArgs)
                or lib.fa_rocm_sizeof_split_plan() != C.sizeof(SplitPlan)):
            raise RuntimeError("libfa_rocm.so argument records do not match this binding")
        _lib = lib
    return _lib


def last_error() -> str:
    return load().fa_rocm_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(last_error())
