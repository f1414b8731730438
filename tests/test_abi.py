"""CPU tests of the drop-in boundary: the shared library loads without a GPU and exports every
symbol include/bz_hip.h declares; the ctypes table covers exactly that set."""
import os
import re

from blitz_scale_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if fn.endswith(".h"):
            text = open(os.path.join(ROOT, "include", fn)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names |= set(re.findall(r"\b(bz_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    decl = declared_symbols()
    assert len(decl) >= 20
    for name in sorted(decl):
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    assert decl == set(_lib.SIGNATURES), (decl ^ set(_lib.SIGNATURES))


def test_identification_and_error_strings_need_no_gpu():
    lib = _lib.load()
    assert b"gfx950" in lib.bz_build_info()
    assert lib.bz_error_string(0) == b"success"
    assert b"workspace" in lib.bz_error_string(_lib.BZ_ERR_WORKSPACE)


def test_layout_strides_and_pool_size():
    lib = _lib.load()
    kv = _lib.BzPagedKV()
    kv.num_kv_heads, kv.page_size, kv.head_dim, kv.kv_dtype = 8, 16, 128, _lib.BZ_BF16
    lib.bz_paged_kv_set_layout(kv, _lib.BZ_LAYOUT_NHD)  # src/kernel/page.h:59-61
    assert (kv.stride_page, kv.stride_n, kv.stride_h) == (2 * 8 * 16 * 128, 8 * 128, 128)
    lib.bz_paged_kv_set_layout(kv, _lib.BZ_LAYOUT_HND)
    assert (kv.stride_page, kv.stride_n, kv.stride_h) == (2 * 8 * 16 * 128, 128, 16 * 128)
    # src/blitz/cache_manager.h:136-142: sizeof(T) * max_pages * (H*P*D) * 2 * layers
    assert lib.bz_kv_pool_bytes(32, 30000, 8, 64, 128, _lib.BZ_F16) == 2 * 30000 * 8 * 64 * 128 * 2 * 32
    lib.bz_kv_layer_view(kv, 1 << 40, 3, 1000)  # layer stride = max_pages * stride_page (llama.h:378-381)
    assert kv.k_data == (1 << 40) + 3 * 1000 * kv.stride_page * 2
    assert kv.v_data == kv.k_data + kv.stride_page  # v = k + H*P*D elements (page.h:42-43)


def test_argument_errors_are_reported_before_anything_touches_a_gpu():
    """Bad arguments come back as BZ_ERR_* codes from the host-side checks (no kernel is launched on a
    null table, an unplanned handle or an unsupported type), so this runs without a GPU."""
    import ctypes as C
    lib = _lib.load()
    kv = _lib.BzPagedKV()
    kv.num_kv_heads, kv.page_size, kv.head_dim, kv.kv_dtype, kv.batch_size = 8, 16, 128, _lib.BZ_BF16, 4
    lib.bz_paged_kv_set_layout(kv, _lib.BZ_LAYOUT_HND)
    fake = C.c_void_p(1 << 20)  # never dereferenced on the host
    assert lib.bz_batch_decode(None, fake, _lib.BZ_BF16, C.byref(kv), fake, _lib.BZ_BF16, 32, 0, 1e4, 0.0, None,
                               None, None, None) == _lib.BZ_ERR_BAD_ARG
    plan = lib.bz_decode_plan_create()
    try:
        assert lib.bz_batch_decode(plan, fake, _lib.BZ_BF16, C.byref(kv), fake, _lib.BZ_BF16, 32, 0, 1e4, 0.0, None,
                                   None, None, None) == _lib.BZ_ERR_NOT_PLANNED
        assert lib.bz_decode_plan(plan, fake, 1 << 20, fake, 1 << 20, None, None, 4, 32, 8, 128, 16, 0,
                                  None) == _lib.BZ_ERR_BAD_ARG
        assert lib.bz_decode_plan_info(plan, None, None, None) == _lib.BZ_ERR_NOT_PLANNED
    finally:
        lib.bz_decode_plan_destroy(plan)
    # page writers: pool pointers set, table pointers cleared (what Stub::forward leaves behind after a step)
    kv.k_data, kv.v_data = 1 << 30, (1 << 30) + 4096
    assert lib.bz_append_decode_kv(C.byref(kv), fake, fake, _lib.BZ_BF16, None, 0, 0, 1e4, None, None,
                                   None) == _lib.BZ_ERR_BAD_ARG
    assert lib.bz_store_prefill_kv(C.byref(kv), fake, fake, _lib.BZ_BF16, None, 16, None, 0, 0, 1e4, None, None,
                                   None) == _lib.BZ_ERR_BAD_ARG
    assert lib.bz_steps_ahead_advance(None, None) == _lib.BZ_ERR_BAD_ARG
    # migration payload: an e4m3 pool cannot travel as bf16
    kv.kv_dtype = _lib.BZ_E4M3
    assert lib.bz_kv_pages_pack(fake, 100, C.byref(kv), fake, 4, 0, 2, fake, _lib.BZ_BF16, None, None,
                                None) == _lib.BZ_ERR_UNSUPPORTED
    assert lib.bz_kv_pages_pack(fake, 100, None, fake, 4, 0, 2, fake, _lib.BZ_E4M3, None, None,
                                None) == _lib.BZ_ERR_BAD_ARG
    # the cached-K conversion: table pointers cleared -> bad argument; an e4m3 pool would be requantised -> unsupported
    assert lib.bz_rope_cached_k(C.byref(kv), 1e4, 0, None) == _lib.BZ_ERR_BAD_ARG
    ids = (C.c_int32 * 8)()
    kv.indices = kv.indptr = kv.last_page_len = C.addressof(ids)
    assert lib.bz_rope_cached_k(C.byref(kv), 1e4, 0, None) == _lib.BZ_ERR_UNSUPPORTED
    assert lib.bz_rope_cached_k(None, 1e4, 0, None) == _lib.BZ_ERR_BAD_ARG
    # prefill plan: the bf16 mode is one of the two named ones; fewer K/V rows than q rows is refused on the host
    pplan = lib.bz_prefill_plan_create()
    try:
        assert lib.bz_prefill_plan_set_bf16_mode(pplan, 2) == _lib.BZ_ERR_BAD_ARG
        assert lib.bz_prefill_plan_set_bf16_mode(pplan, _lib.BZ_PREFILL_BF16_HEAD_TAIL) == 0
        qo, kvp = (C.c_int32 * 2)(0, 10), (C.c_int32 * 2)(0, 9)
        fb, ib = C.c_size_t(), C.c_size_t()
        assert lib.bz_prefill_plan_workspace(pplan, qo, kvp, 1, 4, 4, 128, C.byref(fb), C.byref(ib)) == _lib.BZ_ERR_UNSUPPORTED
        kvp[1] = 30
        assert lib.bz_prefill_plan_workspace(pplan, qo, kvp, 1, 4, 4, 128, C.byref(fb), C.byref(ib)) == 0
        assert fb.value == 30 * 512 and ib.value == 256  # the angle table covers the K/V length; one job of 32 bytes
    finally:
        lib.bz_prefill_plan_destroy(pplan)
