"""ctypes front end of the CPU checker (oracle/bz_oracle.c).  TEST INFRASTRUCTURE ONLY:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the
product.  Arrays are numpy: uint16 bits for f16/bf16, uint8 bits for e4m3, int32 page tables.

Everything numeric goes through the C file; the KV migration wire format (kv_pages_pack /
kv_pages_unpack) is byte and index work and is stated here in numpy, following
src/blitz/migration_manager.h:86-92 (page addressing) and :455-467 (message order).  Every function
is pinned by independent checks in tests/ (closed forms, float64 dense implementations, library
routines, literal walks of the reference's loops); none is "parity unpinned" except, for all of them,
agreement with the reference's private FlashInfer fork, whose source is not in the checkout.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
F16, BF16, E4M3, F32 = 0, 1, 2, 3
ROPE_NONE, ROPE_Q_ONLY, ROPE_FULL = 0, 1, 2


class _PagedKV(C.Structure):
    _fields_ = [("k_base", C.c_void_p), ("v_base", C.c_void_p), ("indices", C.c_void_p), ("indptr", C.c_void_p),
                ("last_page_len", C.c_void_p), ("batch_size", C.c_int32), ("page_size", C.c_int32),
                ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32), ("stride_page", C.c_int64),
                ("stride_n", C.c_int64), ("stride_h", C.c_int64), ("kv_dtype", C.c_int32)]


def build(force=False):
    """gcc the checker (both the scalar and the OpenMP build)."""
    if force or not all(os.path.exists(os.path.join(HERE, n)) for n in ("libbz_oracle.so", "libbz_oracle_omp.so")):
        subprocess.check_call(["make", "-C", HERE, "-B" if force else "-s", "all"], stdout=subprocess.DEVNULL)


_libs = {}


def lib(parallel=False):
    name = "libbz_oracle_omp.so" if parallel else "libbz_oracle.so"
    if name not in _libs:
        build()
        l = C.CDLL(os.path.join(HERE, name))
        l.bzo_f16_to_f32.restype = C.c_float
        l.bzo_f16_to_f32.argtypes = [C.c_uint16]
        l.bzo_bf16_to_f32.restype = C.c_float
        l.bzo_bf16_to_f32.argtypes = [C.c_uint16]
        l.bzo_e4m3_to_f32.restype = C.c_float
        l.bzo_e4m3_to_f32.argtypes = [C.c_uint8]
        l.bzo_f32_to_f16.restype = C.c_uint16
        l.bzo_f32_to_f16.argtypes = [C.c_float]
        l.bzo_f32_to_bf16.restype = C.c_uint16
        l.bzo_f32_to_bf16.argtypes = [C.c_float]
        l.bzo_f32_to_e4m3.restype = C.c_uint8
        l.bzo_f32_to_e4m3.argtypes = [C.c_float]
        l.bzo_num_threads.restype = C.c_int
        _libs[name] = l
    return _libs[name]


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def storage_np(dtype):
    return {F16: np.uint16, BF16: np.uint16, E4M3: np.uint8, F32: np.float32}[dtype]


def to_f32(bits, dtype):
    bits = _c(bits, storage_np(dtype))
    out = np.empty(bits.shape, np.float32)
    lib().bzo_to_f32(_p(bits), dtype, C.c_size_t(bits.size), _p(out))
    return out


def from_f32(x, dtype):
    x = _c(x, np.float32)
    out = np.empty(x.shape, storage_np(dtype))
    lib().bzo_from_f32(_p(x), dtype, C.c_size_t(x.size), _p(out))
    return out


def rope_freqs(D, theta):
    f = np.empty(D // 2, np.float32)
    lib().bzo_rope_freqs(D, C.c_float(theta), _p(f))
    return f


def rope_llama(x, pos, theta):
    """x: fp32 [D]; returns the rotated copy."""
    y = _c(x, np.float32).copy()
    lib().bzo_rope_llama(_p(y), y.shape[-1], int(pos), C.c_float(theta))
    return y


class PagedKV:
    """One layer plane of a pool (numpy storage bits) plus its page table.

    k_pool / v_pool are flat arrays addressed page*stride_page + slot*stride_n + head*stride_h + d;
    they may be two views of one buffer (v offset by stride_page/2, src/kernel/page.h:42-43).
    """

    def __init__(self, k_pool, v_pool, indices, indptr, last_page_len, page_size, num_kv_heads, head_dim,
                 stride_page, stride_n, stride_h, kv_dtype):
        self.k_pool, self.v_pool = k_pool, v_pool
        self.indices, self.indptr = _c(indices, np.int32), _c(indptr, np.int32)
        self.last_page_len = _c(last_page_len, np.int32)
        self.batch_size = len(self.last_page_len)
        self.page_size, self.num_kv_heads, self.head_dim = page_size, num_kv_heads, head_dim
        self.stride_page, self.stride_n, self.stride_h = stride_page, stride_n, stride_h
        self.kv_dtype = kv_dtype
        assert k_pool.flags.c_contiguous or k_pool.ndim == 1
        assert k_pool.dtype == storage_np(kv_dtype) and v_pool.dtype == storage_np(kv_dtype)

    def struct(self):
        s = _PagedKV()
        s.k_base, s.v_base = self.k_pool.ctypes.data, self.v_pool.ctypes.data
        s.indices, s.indptr = self.indices.ctypes.data, self.indptr.ctypes.data
        s.last_page_len = self.last_page_len.ctypes.data
        s.batch_size, s.page_size = self.batch_size, self.page_size
        s.num_kv_heads, s.head_dim = self.num_kv_heads, self.head_dim
        s.stride_page, s.stride_n, s.stride_h = self.stride_page, self.stride_n, self.stride_h
        s.kv_dtype = self.kv_dtype
        return s

    def seq_lens(self):
        out = np.empty(self.batch_size, np.int64)
        s = self.struct()
        lib().bzo_seq_lens(C.byref(s), _p(out))
        return out


def batch_decode(q_bits, q_dtype, kv, num_qo_heads, rope_mode=ROPE_NONE, rope_theta=1e4, sm_scale=None,
                 k_scale=None, v_scale=None, want_lse=False, parallel=False):
    """fp32 [B, Hq, D] (and the natural-log lse [B, Hq] when asked)."""
    q_bits = _c(q_bits, storage_np(q_dtype))
    D = kv.head_dim
    if sm_scale is None:
        sm_scale = 1.0 / np.sqrt(D)
    out = np.empty((kv.batch_size, num_qo_heads, D), np.float32)
    lse = np.empty((kv.batch_size, num_qo_heads), np.float32) if want_lse else None
    ks, vs = _c(k_scale, np.float32), _c(v_scale, np.float32)
    s = kv.struct()
    lib(parallel).bzo_batch_decode(_p(q_bits), q_dtype, C.byref(s), num_qo_heads, rope_mode, C.c_float(rope_theta),
                                   C.c_float(sm_scale), _p(ks), _p(vs), _p(out), _p(lse))
    return (out, lse) if want_lse else out


def batch_prefill_ragged(q_bits, k_bits, v_bits, dtype, indptr, Hq, Hkv, D, causal=True, rope=False,
                         rope_theta=1e4, sm_scale=None, rows=None, parallel=False):
    """fp32 [N or len(rows), Hq, D].  rope: False / True rotate neither / both of q and k at their offsets inside
    the request (in fp32, nothing is rounded); "q" rotates q only (k rows hold rotated K already)."""
    q_bits, k_bits, v_bits = (_c(a, storage_np(dtype)) for a in (q_bits, k_bits, v_bits))
    indptr = _c(indptr, np.int32)
    B = len(indptr) - 1
    if sm_scale is None:
        sm_scale = 1.0 / np.sqrt(D)
    rows = _c(rows, np.int32)
    n = int(indptr[-1]) if rows is None else len(rows)
    out = np.empty((n, Hq, D), np.float32)
    lib(parallel).bzo_batch_prefill_ragged(_p(q_bits), _p(k_bits), _p(v_bits), dtype, _p(indptr), B, Hq, Hkv, D,
                                           int(causal), 2 if rope == "q" else int(bool(rope)), C.c_float(rope_theta),
                                           C.c_float(sm_scale),
                                           _p(rows), 0 if rows is None else len(rows), _p(out))
    return out


def store_prefill_kv(kv, k_bits, v_bits, src_dtype, ragged_indptr, rope=False, rope_theta=1e4, k_scale=None,
                     v_scale=None):
    """Writes into kv.k_pool / kv.v_pool in place."""
    k_bits, v_bits = _c(k_bits, storage_np(src_dtype)), _c(v_bits, storage_np(src_dtype))
    ri = _c(ragged_indptr, np.int32)
    ks, vs = _c(k_scale, np.float32), _c(v_scale, np.float32)
    s = kv.struct()
    lib().bzo_store_prefill_kv(C.byref(s), _p(k_bits), _p(v_bits), src_dtype, _p(ri), int(rope), C.c_float(rope_theta),
                               _p(ks), _p(vs))


def append_decode_kv(kv, k_bits, v_bits, src_dtype, rope=False, rope_theta=1e4, k_scale=None, v_scale=None):
    k_bits, v_bits = _c(k_bits, storage_np(src_dtype)), _c(v_bits, storage_np(src_dtype))
    ks, vs = _c(k_scale, np.float32), _c(v_scale, np.float32)
    s = kv.struct()
    lib().bzo_append_decode_kv(C.byref(s), _p(k_bits), _p(v_bits), src_dtype, int(rope), C.c_float(rope_theta),
                               _p(ks), _p(vs))


def rope_decode_q(q_bits, dtype, kv, Hq, theta):
    q = _c(q_bits, storage_np(dtype)).copy()
    s = kv.struct()
    lib().bzo_rope_decode_q_inplace(_p(q), dtype, C.byref(s), Hq, C.c_float(theta))
    return q


def rope_ragged(x_bits, dtype, indptr, H, D, theta):
    x = _c(x_bits, storage_np(dtype)).copy()
    ip = _c(indptr, np.int32)
    lib().bzo_rope_ragged_inplace(_p(x), dtype, _p(ip), len(ip) - 1, H, D, C.c_float(theta))
    return x


def rms_norm(x_bits, w_bits, dtype, eps=1e-5):
    x_bits, w_bits = _c(x_bits, np.uint16), _c(w_bits, np.uint16)
    N, h = x_bits.shape
    out = np.empty((N, h), np.float32)
    lib().bzo_rms_norm(_p(x_bits), _p(w_bits), dtype, N, h, C.c_float(eps), _p(out))
    return out


def add_rms_norm(in_bits, res_bits, w_bits, dtype, eps=1e-5):
    """Returns (normalised fp32, new residual bits)."""
    in_bits, w_bits = _c(in_bits, np.uint16), _c(w_bits, np.uint16)
    res = _c(res_bits, np.uint16).copy()
    N, h = in_bits.shape
    out = np.empty((N, h), np.float32)
    lib().bzo_add_rms_norm(_p(in_bits), _p(res), _p(w_bits), dtype, N, h, C.c_float(eps), _p(out))
    return out, res


def silu_and_mul(in_bits, dtype):
    in_bits = _c(in_bits, np.uint16)
    N, I2 = in_bits.shape
    out = np.empty((N, I2 // 2), np.float32)
    lib().bzo_silu_and_mul(_p(in_bits), dtype, N, I2 // 2, _p(out))
    return out


def add_residual(in_bits, res_bits, dtype):
    in_bits = _c(in_bits, np.uint16)
    res = _c(res_bits, np.uint16).copy()
    lib().bzo_add_residual(_p(in_bits), _p(res), dtype, C.c_size_t(res.size))
    return res


def embedding(token_ids, weight_bits, out_rows=None, out_loc=None):
    """out[loc] = weight[token_ids[t]]; returns the output (rows not written stay zero)."""
    ids = _c(token_ids, np.uint32)
    w = _c(weight_bits, np.uint16)
    hidden = w.shape[1]
    out = np.zeros((len(ids) if out_rows is None else out_rows, hidden), np.uint16)
    loc = _c(out_loc, np.int32) if out_loc is not None else None
    lib().bzo_embedding(_p(out), _p(ids), _p(loc) if loc is not None else None, _p(w), C.c_size_t(len(ids)),
                        C.c_size_t(hidden))
    return out


def gather_last_token(tokens_bits, ragged_indptr):
    t = _c(tokens_bits, np.uint16)
    ip = _c(ragged_indptr, np.int32)
    out = np.empty((len(ip) - 1, t.shape[1]), np.uint16)
    lib().bzo_gather_last_token(_p(out), _p(t), _p(ip), C.c_size_t(len(ip) - 1), C.c_size_t(t.shape[1]))
    return out


def batch_find_max(input_bits, dtype):
    x = _c(input_bits, np.uint16)
    out = np.empty(x.shape[0], np.uint32)
    lib().bzo_batch_find_max(_p(out), _p(x), dtype, C.c_size_t(x.shape[0]), C.c_size_t(x.shape[1]))
    return out


def _wire_scales(kv_dtype, wire_dtype, stride_page, stride_h, Hkv, layer_cnt, k_scale, v_scale):
    """Per-element scale of one (page, layer) chunk for every layer: [layer_cnt][stride_page] fp32, or None."""
    if wire_dtype == kv_dtype or (k_scale is None and v_scale is None):
        return None
    half = stride_page // 2
    head = (np.arange(half) // stride_h) % Hkv
    ks = np.ones((layer_cnt, Hkv), np.float32) if k_scale is None else _c(k_scale, np.float32).reshape(layer_cnt, Hkv)
    vs = np.ones((layer_cnt, Hkv), np.float32) if v_scale is None else _c(v_scale, np.float32).reshape(layer_cnt, Hkv)
    return np.concatenate([ks[:, head], vs[:, head]], axis=1)


def kv_pages_pack(pool_bits, kv_dtype, max_pages, stride_page, page_ids, start_layer, layer_cnt, wire_dtype=None,
                  num_kv_heads=1, stride_h=1, k_scale=None, v_scale=None):
    """The byte stream MigrationManager::send_multi_layer_fast sends (src/blitz/migration_manager.h:455-467):
    for every page in order, for every layer, the stride_page elements at get_page_ptr (:86-92) =
    base + layer*max_pages*stride_page + page*stride_page.  With an e4m3 wire on a 16-bit pool every
    element travels as e4m3(x / scale[layer][head])."""
    pool = _c(pool_bits, storage_np(kv_dtype)).reshape(-1)
    wire_dtype = kv_dtype if wire_dtype is None else wire_dtype
    sc = _wire_scales(kv_dtype, wire_dtype, stride_page, stride_h, num_kv_heads, layer_cnt, k_scale, v_scale)
    out = []
    for page in np.asarray(page_ids, np.int64):
        for l in range(layer_cnt):
            off = ((start_layer + l) * max_pages + int(page)) * stride_page
            chunk = pool[off:off + stride_page]
            if wire_dtype != kv_dtype:
                x = to_f32(chunk, kv_dtype)
                if sc is not None:
                    x = (x / sc[l]).astype(np.float32)
                chunk = from_f32(x, wire_dtype)
            out.append(chunk)
    if not out:
        return np.empty(0, storage_np(wire_dtype))
    return np.concatenate(out)


def kv_pages_unpack(pool_bits, kv_dtype, max_pages, stride_page, page_ids, start_layer, layer_cnt, wire_bits,
                    wire_dtype=None, num_kv_heads=1, stride_h=1, k_scale=None, v_scale=None):
    """The receiving side, in place on pool_bits: message (i, l) goes to page page_ids[i] of layer start_layer + l."""
    pool = pool_bits.reshape(-1)
    wire_dtype = kv_dtype if wire_dtype is None else wire_dtype
    wire = _c(wire_bits, storage_np(wire_dtype)).reshape(-1)
    sc = _wire_scales(kv_dtype, wire_dtype, stride_page, stride_h, num_kv_heads, layer_cnt, k_scale, v_scale)
    c = 0
    for page in np.asarray(page_ids, np.int64):
        for l in range(layer_cnt):
            chunk = wire[c * stride_page:(c + 1) * stride_page]
            if wire_dtype != kv_dtype:
                x = to_f32(chunk, wire_dtype)
                if sc is not None:
                    x = (x * sc[l]).astype(np.float32)
                chunk = from_f32(x, kv_dtype)
            off = ((start_layer + l) * max_pages + int(page)) * stride_page
            pool[off:off + stride_page] = chunk
            c += 1
    return pool_bits


def gemm_strided_batched(a_bits, b_bits, dtype, m, n, k, transa=False, transb=False, alpha=1.0, beta=0.0, c_bits=None,
                         stride_a=None, stride_b=None, stride_c=None, batch=1, parallel=False):
    """Row-major C[b] = alpha op(A[b]) op(B[b]) + beta C[b] with the argument meaning of
    util::CublasWrapper::gemmStridedBatched (src/util/cublas_wrapper.h:33-88); returns C's storage bits."""
    stride_a = m * k if stride_a is None else stride_a
    stride_b = k * n if stride_b is None else stride_b
    stride_c = m * n if stride_c is None else stride_c
    a, b = _c(a_bits, storage_np(dtype)), _c(b_bits, storage_np(dtype))
    need_c = (batch - 1) * stride_c + m * n
    c = np.zeros(need_c, storage_np(dtype)) if c_bits is None else _c(c_bits, storage_np(dtype)).reshape(-1).copy()
    assert c.size >= need_c
    fn = lib(parallel).bzo_gemm_strided_batched
    fn.restype = None
    fn.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                   C.c_float, C.c_void_p, C.c_int64, C.c_int, C.c_int]
    fn(int(transa), int(transb), m, n, k, alpha, _p(a), stride_a, _p(b), stride_b, beta, _p(c), stride_c, batch, dtype)
    return c


def prefill_reservation(lens, page_size):
    lens = _c(lens, np.int32)
    B = len(lens)
    indptr, lpl = np.empty(B + 1, np.int32), np.empty(B, np.int32)
    lib().bzo_prefill_reservation(_p(lens), B, page_size, _p(indptr), _p(lpl))
    return indptr, lpl


def first_fit(free_mask, n):
    """Lowest n free page ids; marks them used.  None (mask untouched) when fewer are free."""
    out = np.empty(max(n, 1), np.int32)
    got = lib().bzo_first_fit(_p(free_mask), len(free_mask), n, _p(out))
    return None if got < n else out[:n].copy()


def table_grow(indices, indptr, last_page_len, page_size, free_mask):
    """One step of growth; returns the new (indices, indptr, last_page_len) or None when out of pages."""
    B = len(last_page_len)
    ind = np.concatenate([_c(indices, np.int32), np.zeros(B + 1, np.int32)])
    ip, lpl = _c(indptr, np.int32).copy(), _c(last_page_len, np.int32).copy()
    n = lib().bzo_table_grow(_p(ind), _p(ip), _p(lpl), B, page_size, _p(free_mask), len(free_mask))
    return None if n < 0 else (ind[:n].copy(), ip, lpl)


def num_threads(parallel=True):
    return lib(parallel).bzo_num_threads()
