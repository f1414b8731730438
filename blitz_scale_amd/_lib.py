"""ctypes binding of the C ABI declared in include/bz_hip.h.

The shared library is the product: there is no Python or CPU fallback.  Loading fails loudly
when blitz_scale_amd/lib/libbz_hip.so has not been built (python -m blitz_scale_amd.build).
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# BZ_HIP_LIB points at another build of the same library (e.g. an experimental kernel variant)
LIB_PATH = os.environ.get("BZ_HIP_LIB") or os.path.join(HERE, "lib", "libbz_hip.so")

BZ_F16, BZ_BF16, BZ_E4M3, BZ_F32 = 0, 1, 2, 3
BZ_ROPE_NONE, BZ_ROPE_Q_ONLY, BZ_ROPE_FULL = 0, 1, 2
BZ_LAYOUT_NHD, BZ_LAYOUT_HND = 0, 1
BZ_NUM_TOKENS_FROM_INDPTR = 0xFFFFFFFF
BZ_PREFILL_BF16_WIDEN_V, BZ_PREFILL_BF16_HEAD_TAIL = 0, 1
BZ_ERR_BAD_ARG, BZ_ERR_UNSUPPORTED, BZ_ERR_WORKSPACE, BZ_ERR_NOT_PLANNED, BZ_ERR_NO_PAGES = 10001, 10002, 10003, 10004, 10005


class BzPagedKV(C.Structure):
    """struct bz_paged_kv (include/bz_hip.h)."""

    _fields_ = [
        ("k_data", C.c_void_p),
        ("v_data", C.c_void_p),
        ("indices", C.c_void_p),
        ("indptr", C.c_void_p),
        ("last_page_len", C.c_void_p),
        ("batch_size", C.c_uint32),
        ("page_size", C.c_uint32),
        ("num_kv_heads", C.c_uint32),
        ("head_dim", C.c_uint32),
        ("stride_page", C.c_uint64),
        ("stride_n", C.c_uint64),
        ("stride_h", C.c_uint64),
        ("kv_dtype", C.c_int32),
        ("reserved", C.c_int32),
        ("steps_ahead", C.c_void_p),
    ]


# name -> (restype, argtypes); every symbol include/bz_hip.h declares
_u32, _i32, _f32, _vp, _sz, _u64 = C.c_uint32, C.c_int, C.c_float, C.c_void_p, C.c_size_t, C.c_uint64
_kvp = C.POINTER(BzPagedKV)
SIGNATURES = {
    "bz_paged_kv_set_layout": (None, [_kvp, _i32]),
    "bz_kv_pool_bytes": (_u64, [_u32, _u64, _u32, _u32, _u32, _i32]),
    "bz_kv_pool_alloc": (_i32, [C.POINTER(_vp), _u64]),
    "bz_kv_pool_free": (_i32, [_vp]),
    "bz_kv_layer_view": (None, [_kvp, _vp, _u32, _u64]),
    "bz_decode_plan_create": (_vp, []),
    "bz_decode_plan_destroy": (None, [_vp]),
    "bz_decode_plan": (_i32, [_vp, _vp, _sz, _vp, _sz, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _vp]),
    "bz_decode_plan_workspace": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _u32, _u32, C.POINTER(_sz),
                                        C.POINTER(_sz)]),
    "bz_decode_plan_host_schedule": (_i32, [_vp, _i32, C.POINTER(_vp), C.POINTER(_sz), C.POINTER(_u32)]),
    "bz_decode_plan_info": (_i32, [_vp, C.POINTER(_u32), C.POINTER(_u32), C.POINTER(_u32)]),
    "bz_decode_plan_step_form": (_i32, [_vp]),
    "bz_decode_plan_set_timing_events": (_i32, [_vp, _vp, _vp]),
    "bz_batch_decode": (_i32, [_vp, _vp, _i32, _kvp, _vp, _i32, _u32, _i32, _f32, _f32, _vp, _vp, _vp, _vp]),
    "bz_decode_step": (_i32, [_vp, _vp, _i32, _vp, _vp, _kvp, _vp, _i32, _u32, _i32, _f32, _f32, _vp, _vp, _vp, _vp]),
    "bz_batch_decode_noalloc_scratch_bytes": (_sz, []),
    "bz_batch_decode_noalloc": (_i32, [_vp, _vp, _i32, _kvp, _vp, _i32, _u32, _i32, _f32, _f32, _vp, _vp, _vp, _vp]),
    "bz_prefill_plan_create": (_vp, []),
    "bz_prefill_plan_destroy": (None, [_vp]),
    "bz_prefill_plan": (_i32, [_vp, _vp, _sz, _vp, _sz, _vp, _vp, _u32, _u32, _u32, _u32, _u32, _vp]),
    "bz_prefill_plan_workspace": (_i32, [_vp, _vp, _vp, _u32, _u32, _u32, _u32, C.POINTER(_sz), C.POINTER(_sz)]),
    "bz_prefill_plan_host_schedule": (_i32, [_vp, C.POINTER(_vp), C.POINTER(_sz), C.POINTER(_u32)]),
    "bz_prefill_plan_set_bf16_mode": (_i32, [_vp, _i32]),
    "bz_prefill_plan_set_timing_events": (_i32, [_vp, _vp, _vp]),
    "bz_rope_cached_k": (_i32, [_vp, _f32, _i32, _vp]),
    "bz_batch_prefill_ragged": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _u32, _u32, _u32, _u32, _i32, _i32,
                                       _f32, _f32, _vp]),
    "bz_store_prefill_kv": (_i32, [_kvp, _vp, _vp, _i32, _vp, _u32, _vp, _u32, _i32, _f32, _vp, _vp, _vp]),
    "bz_append_decode_kv": (_i32, [_kvp, _vp, _vp, _i32, _vp, _u32, _i32, _f32, _vp, _vp, _vp]),
    "bz_steps_ahead_advance": (_i32, [_vp, _vp]),
    "bz_rms_norm": (_i32, [_vp, _vp, _vp, _i32, _u32, _u32, _f32, _vp]),
    "bz_add_rms_norm": (_i32, [_vp, _vp, _vp, _i32, _u32, _u32, _f32, _vp]),
    "bz_silu_and_mul": (_i32, [_vp, _vp, _i32, _u32, _u32, _vp]),
    "bz_add_residual": (_i32, [_vp, _vp, _i32, _u32, _u32, _vp]),
    "bz_embedding": (_i32, [_vp, _vp, _vp, _vp, _i32, _u32, _u32, _vp]),
    "bz_gather_last_token": (_i32, [_vp, _vp, _vp, _i32, _u32, _u32, _u32, _vp]),
    "bz_batch_find_max": (_i32, [_vp, _vp, _i32, _u32, _u32, _vp]),
    "bz_kv_wire_bytes": (_u64, [_u32, _u32, _kvp, _i32]),
    "bz_kv_pages_pack": (_i32, [_vp, _u64, _kvp, _vp, _u32, _u32, _u32, _vp, _i32, _vp, _vp, _vp]),
    "bz_kv_pages_unpack": (_i32, [_vp, _u64, _kvp, _vp, _u32, _u32, _u32, _vp, _i32, _vp, _vp, _vp]),
    "bz_cm_create": (_i32, [C.POINTER(_vp), _u32, _u32, _u32, _u32, _u32, _i32, _i32, _i32]),
    "bz_cm_destroy": (None, [_vp]),
    "bz_cm_batch_prefill": (_i32, [_vp, _vp, _u32, C.POINTER(_i32)]),
    "bz_cm_batch_grow": (_i32, [_vp, _i32]),
    "bz_cm_batch_filter": (_i32, [_vp, _i32, _vp, _u32]),
    "bz_cm_batch_extend": (_i32, [_vp, _i32, _i32]),
    "bz_cm_batch_release": (_i32, [_vp, _i32]),
    "bz_cm_batch_table": (_i32, [_vp, _i32, C.POINTER(_vp), C.POINTER(_u32), C.POINTER(_vp), C.POINTER(_vp),
                                 C.POINTER(_u32)]),
    "bz_cm_stats": (_i32, [_vp, C.POINTER(_u64), C.POINTER(_u64), C.POINTER(_u64)]),
    "bz_cm_pool": (_i32, [_vp, C.POINTER(_vp), C.POINTER(_u64)]),
    "bz_build_info": (C.c_char_p, []),
    "bz_error_string": (C.c_char_p, [_i32]),
}

_lib = None


def load():
    """Load libbz_hip.so and attach the signatures.  Raises if the library is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the HIP library first (python -m blitz_scale_amd.build). "
            "There is no fallback implementation."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class BzError(RuntimeError):
    """Mirror of the std::runtime_error the reference wrappers throw on a non-zero status."""


def check(code, what):
    if code != 0:
        msg = load().bz_error_string(code).decode()
        raise BzError(f"{what} error: {msg} ({code})")
