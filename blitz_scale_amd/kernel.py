"""Host-side mirror of the reference's `blitz::kernel` interface over the C ABI.

Names, argument order and error behaviour follow src/kernel/{page,attention,rms_norm,activation,
add,flashinfer_types}.h of the BlitzScale worker; torch tensors stand in for the raw device
pointers the C++ callers pass (torch is only the allocator here: every function hands
`tensor.data_ptr()` to libbz_hip.so).  Trailing keyword arguments are the parameters the
reference never exposes (RoPE theta, softmax scale, fp8 scales, stream).
"""
import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import (BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_FULL, BZ_ROPE_NONE,
                   BZ_ROPE_Q_ONLY, BzError, BzPagedKV, check)

_DTYPES = {torch.float16: BZ_F16, torch.bfloat16: BZ_BF16, torch.float32: BZ_F32, torch.uint8: BZ_E4M3}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPES[torch.float8_e4m3fn] = BZ_E4M3


def bz_dtype(t):
    return _DTYPES[t.dtype if isinstance(t, torch.Tensor) else t]


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        return C.c_void_p(t.data_ptr())
    return C.c_void_p(int(t))


def _stream(stream):
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    return C.c_void_p(int(stream))


def _host_i32(a):
    if isinstance(a, torch.Tensor):
        a = a.cpu().numpy()
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


class PageTable:
    """blitz::kernel::PageTable<DType, IdType> (src/kernel/page.h:12-64).

    base: torch tensor holding (at least) one layer plane of the pool, element type = KV dtype.
    layout: BZ_LAYOUT_NHD is the reference's in-page order, BZ_LAYOUT_HND the re-laid-out one.
    """

    def __init__(self, batch_size, page_size, num_heads, head_size, base, layout=BZ_LAYOUT_HND):
        self.indices, self.indptr, self.last_page_len = [], [], []
        self.batch_size = batch_size
        self.page_size, self.num_heads, self.head_size = page_size, num_heads, head_size
        self.layout = layout
        self.base = base
        self.kv_dtype = bz_dtype(base)
        self.elem_bytes = base.element_size()
        self.stride_page = 2 * num_heads * page_size * head_size
        if layout == BZ_LAYOUT_HND:
            self.stride_n, self.stride_h = head_size, page_size * head_size
        else:
            self.stride_n, self.stride_h = num_heads * head_size, head_size
        self.k_data = base.data_ptr()
        self.v_data = self.k_data + (self.stride_page // 2) * self.elem_bytes
        self.indices_d = self.indptr_d = self.last_page_len_d = None
        self.steps_ahead_d = None  # optional device int32: the table is this many decode steps ahead of the present

    def set_layer(self, layer, max_num_pages):
        """The per-layer pointer bump of src/model/llama.h:378-381, as an absolute view."""
        self.k_data = self.base.data_ptr() + layer * max_num_pages * self.stride_page * self.elem_bytes
        self.v_data = self.k_data + (self.stride_page // 2) * self.elem_bytes

    def upload(self, device="cuda"):
        """One blob [indices | indptr | last_page_len] like Stub::forward (src/blitz/stub.h:1288-1313)."""
        blob = np.concatenate([_host_i32(self.indices), _host_i32(self.indptr), _host_i32(self.last_page_len)])
        host = torch.from_numpy(blob)
        prev = getattr(self, "_blob_d", None)
        if prev is not None and prev.numel() == host.numel() and prev.device.type == torch.device(device).type:
            prev.copy_(host)  # same device buffer: addresses recorded into a HIP graph stay valid
        else:
            self._blob_d = host.to(device)
        n0, n1 = len(self.indices), len(self.indptr)
        self.indices_d = self._blob_d[:n0]
        self.indptr_d = self._blob_d[n0:n0 + n1]
        self.last_page_len_d = self._blob_d[n0 + n1:]
        return self

    def seq_lens(self):
        ip, lp = _host_i32(self.indptr), _host_i32(self.last_page_len)
        n = ip[1:] - ip[:-1]
        return np.where(n > 0, (n - 1) * self.page_size + lp, 0)

    def as_struct(self):
        s = BzPagedKV()
        s.k_data, s.v_data = self.k_data, self.v_data
        s.indices = self.indices_d.data_ptr() if self.indices_d is not None else None
        s.indptr = self.indptr_d.data_ptr() if self.indptr_d is not None else None
        s.last_page_len = self.last_page_len_d.data_ptr() if self.last_page_len_d is not None else None
        s.batch_size, s.page_size = self.batch_size, self.page_size
        s.num_kv_heads, s.head_dim = self.num_heads, self.head_size
        s.stride_page, s.stride_n, s.stride_h = self.stride_page, self.stride_n, self.stride_h
        s.kv_dtype = self.kv_dtype
        s.steps_ahead = self.steps_ahead_d.data_ptr() if self.steps_ahead_d is not None else None
        return s


class BlitzBatchDecodeHandler:
    """blitz::kernel::BlitzBatchDecodeHandler (src/kernel/flashinfer_types.h:44-72)."""

    def __init__(self):
        self._h = _lib.load().bz_decode_plan_create()  # create_flashinfer_decode_handler()

    def get(self):
        return self._h

    def empty(self):
        return not self._h

    def plan(self, float_buffer, float_buffer_size, int_buffer, int_buffer_size, indptr_h, last_page_len_h,
             batch_size, num_qo_heads, num_kv_heads, head_dim, page_size, *, split_tokens=0, stream=None):
        ip, lp = _host_i32(indptr_h), _host_i32(last_page_len_h)
        rc = _lib.load().bz_decode_plan(self._h, _ptr(float_buffer), float_buffer_size, _ptr(int_buffer),
                                        int_buffer_size, ip.ctypes.data_as(C.c_void_p),
                                        lp.ctypes.data_as(C.c_void_p), batch_size, num_qo_heads, num_kv_heads,
                                        head_dim, page_size, split_tokens, _stream(stream))
        check(rc, "Handler plan")
        self._keep = (float_buffer, int_buffer)

    def workspace(self, indptr_h, last_page_len_h, batch_size, num_qo_heads, num_kv_heads, head_dim, page_size, *,
                  split_tokens=0, num_compute_units=0):
        """(float_buffer_bytes, int_buffer_bytes) plan() would use for this batch; no GPU needed when
        num_compute_units is given."""
        ip, lp = _host_i32(indptr_h), _host_i32(last_page_len_h)
        fb, ib = C.c_size_t(), C.c_size_t()
        check(_lib.load().bz_decode_plan_workspace(self._h, ip.ctypes.data_as(C.c_void_p), lp.ctypes.data_as(C.c_void_p),
                                                   batch_size, num_qo_heads, num_kv_heads, head_dim, page_size,
                                                   split_tokens, num_compute_units, C.byref(fb), C.byref(ib)),
              "Handler workspace")
        return fb.value, ib.value

    def host_schedule(self, which):
        """numpy copy [records, ints] of one table of the last schedule (see bz_decode_plan_host_schedule)."""
        data, n, k = C.c_void_p(), C.c_size_t(), C.c_uint32()
        check(_lib.load().bz_decode_plan_host_schedule(self._h, which, C.byref(data), C.byref(n), C.byref(k)),
              "Handler schedule")
        if n.value == 0:
            return np.zeros((0, max(k.value, 1)), np.int32)
        buf = (C.c_int32 * (n.value * k.value)).from_address(data.value)
        return np.frombuffer(buf, np.int32).reshape(n.value, k.value).copy()

    def set_timing_events(self, start=None, stop=None):
        """hipEvent_t handles recorded right before / after the decode kernel launch (None: off)."""
        check(_lib.load().bz_decode_plan_set_timing_events(self._h, start, stop), "Handler timing events")

    def info(self):
        a, b, c = C.c_uint32(), C.c_uint32(), C.c_uint32()
        check(_lib.load().bz_decode_plan_info(self._h, C.byref(a), C.byref(b), C.byref(c)), "Handler info")
        return {"segments": a.value, "split_seqs": b.value, "workgroups": c.value}

    def step_form(self):
        """'one_call': decode_step on this plan runs its two-launch form; 'two_calls': it runs the append and
        the decode one after the other (the faster order where most (sequence, kv head)s are not split)."""
        rc = _lib.load().bz_decode_plan_step_form(self._h)
        check(min(rc, 0), "Handler step form")
        return "one_call" if rc == 1 else "two_calls"

    def __del__(self):
        try:
            if self._h:
                _lib.load().bz_decode_plan_destroy(self._h)
        except Exception:
            pass


class BatchPrefillRaggedHandler:
    """blitz::kernel::BatchPrefillRaggedHandler (src/kernel/flashinfer_types.h:12-41)."""

    def __init__(self):
        self._h = _lib.load().bz_prefill_plan_create()  # create_flashinfer_prefill_handler()

    def get(self):
        return self._h

    def empty(self):
        return not self._h

    def plan(self, float_buffer, float_buffer_size, int_buffer, int_buffer_size, qo_indptr_h, kv_indptr_h,
             batch_size, num_qo_heads, num_kv_heads, head_dim, page_size, *, stream=None):
        qo, kv = _host_i32(qo_indptr_h), _host_i32(kv_indptr_h)
        rc = _lib.load().bz_prefill_plan(self._h, _ptr(float_buffer), float_buffer_size, _ptr(int_buffer),
                                         int_buffer_size, qo.ctypes.data_as(C.c_void_p),
                                         kv.ctypes.data_as(C.c_void_p), batch_size, num_qo_heads, num_kv_heads,
                                         head_dim, page_size, _stream(stream))
        check(rc, "Handler plan")
        self._keep = (float_buffer, int_buffer)

    def workspace(self, qo_indptr_h, kv_indptr_h, batch_size, num_qo_heads, num_kv_heads, head_dim):
        """(float_buffer_bytes, int_buffer_bytes) plan() would use; host only."""
        qo, kv = _host_i32(qo_indptr_h), _host_i32(kv_indptr_h)
        fb, ib = C.c_size_t(), C.c_size_t()
        check(_lib.load().bz_prefill_plan_workspace(self._h, qo.ctypes.data_as(C.c_void_p),
                                                    kv.ctypes.data_as(C.c_void_p), batch_size, num_qo_heads,
                                                    num_kv_heads, head_dim, C.byref(fb), C.byref(ib)),
              "Handler workspace")
        return fb.value, ib.value

    def set_timing_events(self, start=None, stop=None):
        """hipEvent_t handles recorded right before / after the attention kernel's launch (None: off)."""
        check(_lib.load().bz_prefill_plan_set_timing_events(self._h, start, stop), "Handler timing events")

    def set_bf16_mode(self, mode):
        """BZ_PREFILL_BF16_WIDEN_V (default) or BZ_PREFILL_BF16_HEAD_TAIL: see include/bz_hip.h."""
        check(_lib.load().bz_prefill_plan_set_bf16_mode(self._h, mode), "Handler bf16 mode")

    def host_schedule(self):
        """numpy copy [workgroups, 8] of the last job list: first q row and q rows of the request (0 = padding), first q
        row of the tile, q head, first K/V row and K/V rows of the request, 0, 0."""
        data, n, k = C.c_void_p(), C.c_size_t(), C.c_uint32()
        check(_lib.load().bz_prefill_plan_host_schedule(self._h, C.byref(data), C.byref(n), C.byref(k)),
              "Handler schedule")
        if n.value == 0:
            return np.zeros((0, 8), np.int32)
        buf = (C.c_int32 * (n.value * k.value)).from_address(data.value)
        return np.frombuffer(buf, np.int32).reshape(n.value, k.value).copy()

    def __del__(self):
        try:
            if self._h:
                _lib.load().bz_prefill_plan_destroy(self._h)
        except Exception:
            pass


def batch_decode_attention(handler, q_input, paged_kv, output, num_qo_heads, *, rope_mode=BZ_ROPE_Q_ONLY,
                           rope_theta=1e4, sm_scale=0.0, k_scale=None, v_scale=None, lse=None, stream=None):
    """src/kernel/attention.h:24-31."""
    s = paged_kv.as_struct()
    rc = _lib.load().bz_batch_decode(handler.get(), _ptr(q_input), bz_dtype(q_input), C.byref(s), _ptr(output),
                                     bz_dtype(output), num_qo_heads, rope_mode, rope_theta, sm_scale, _ptr(k_scale),
                                     _ptr(v_scale), _ptr(lse), _stream(stream))
    check(rc, "batchDecodeAttention")


def decode_step(handler, q_input, k_new, v_new, paged_kv, output, num_qo_heads, *, rope=True, rope_theta=1e4,
                sm_scale=0.0, k_scale=None, v_scale=None, lse=None, stream=None):
    """append_decode_kv_cache followed by batch_decode_attention (src/layer/attn.h:196-203) as one call: the
    new K (rotated when rope) and V rows go into the cache, q is rotated inside the kernels and left as it is."""
    s = paged_kv.as_struct()
    rc = _lib.load().bz_decode_step(handler.get(), _ptr(q_input), bz_dtype(q_input), _ptr(k_new), _ptr(v_new), C.byref(s),
                                    _ptr(output), bz_dtype(output), num_qo_heads, int(rope), rope_theta, sm_scale,
                                    _ptr(k_scale), _ptr(v_scale), _ptr(lse), _stream(stream))
    check(rc, "decodeStep")


def batch_decode_attention_noalloc(handler, q_input, paged_kv, output, num_qo_heads, *, rope_mode=BZ_ROPE_Q_ONLY,
                                   rope_theta=1e4, sm_scale=0.0, k_scale=None, v_scale=None, lse=None, stream=None):
    """batch_decode_attention with the split-K partials in the library's own fixed device array instead of
    the plan's float workspace: the call allocates nothing (no counterpart in the reference)."""
    s = paged_kv.as_struct()
    rc = _lib.load().bz_batch_decode_noalloc(handler.get(), _ptr(q_input), bz_dtype(q_input), C.byref(s),
                                             _ptr(output), bz_dtype(output), num_qo_heads, rope_mode, rope_theta,
                                             sm_scale, _ptr(k_scale), _ptr(v_scale), _ptr(lse), _stream(stream))
    check(rc, "batchDecodeAttention")


def batch_prefill_attention(handler, q_input, qo_indptr, k_input, v_input, kv_indptr, output, batch_size,
                            num_qo_heads, num_kv_heads, head_size, *, causal=True, rope_mode=BZ_ROPE_NONE,
                            rope_theta=1e4, sm_scale=0.0, stream=None):
    """src/kernel/attention.h:9-22."""
    rc = _lib.load().bz_batch_prefill_ragged(handler.get(), _ptr(q_input), _ptr(qo_indptr), _ptr(k_input),
                                             _ptr(v_input), _ptr(kv_indptr), _ptr(output), bz_dtype(q_input),
                                             batch_size, num_qo_heads, num_kv_heads, head_size, int(causal),
                                             rope_mode, rope_theta, sm_scale, _stream(stream))
    check(rc, "BatchPrefillWithRaggedKVCache")


def store_prefill_kv_cache(page_table, k_data, v_data, ragged_indptr, *, num_tokens=None, q=None, num_qo_heads=0,
                           rope=False, rope_theta=1e4, k_scale=None, v_scale=None, stream=None):
    """src/kernel/page.h:66-67."""
    if num_tokens is None:
        num_tokens = k_data.shape[0]
    s = page_table.as_struct()
    rc = _lib.load().bz_store_prefill_kv(C.byref(s), _ptr(k_data), _ptr(v_data), bz_dtype(k_data),
                                         _ptr(ragged_indptr), num_tokens, _ptr(q), num_qo_heads, int(rope),
                                         rope_theta, _ptr(k_scale), _ptr(v_scale), _stream(stream))
    check(rc, "AppendPagedKVCache")


def append_decode_kv_cache(page_table, k_data, v_data, *, q=None, num_qo_heads=0, rope=False, rope_theta=1e4,
                           k_scale=None, v_scale=None, stream=None):
    """src/kernel/page.h:69-70."""
    s = page_table.as_struct()
    rc = _lib.load().bz_append_decode_kv(C.byref(s), _ptr(k_data), _ptr(v_data), bz_dtype(k_data), _ptr(q),
                                         num_qo_heads, int(rope), rope_theta, _ptr(k_scale), _ptr(v_scale),
                                         _stream(stream))
    check(rc, "AppendPagedKVCacheDecode")


def rope_cached_k(page_table, *, rope_theta=1e4, inverse=False, stream=None):
    """Rotate (or un-rotate) the cached K rows of every sequence of the table in place: a cache filled under the
    reference's raw-K convention (kRoPELlama at every decode call, src/kernel/attention_decode.cu:35) converted once
    to the rotated-K convention of the fast decode path, or back.  No counterpart in the reference."""
    s = page_table.as_struct()
    check(_lib.load().bz_rope_cached_k(C.byref(s), rope_theta, int(inverse), _stream(stream)), "ropeCachedK")


def steps_ahead_advance(steps_ahead, *, stream=None):
    """End of a decode step under a page table that runs ahead of the present: counter -= 1, not below 0."""
    check(_lib.load().bz_steps_ahead_advance(_ptr(steps_ahead), _stream(stream)), "stepsAheadAdvance")


def rms_norm(input, weight, output, num_tokens, hidden_size, eps=1e-5, *, stream=None):
    """src/kernel/rms_norm.h:11-19."""
    rc = _lib.load().bz_rms_norm(_ptr(input), _ptr(weight), _ptr(output), bz_dtype(input), num_tokens, hidden_size,
                                 eps, _stream(stream))
    check(rc, "rmsNorm")


def add_rms_norm(input, residual, weight, num_tokens, hidden_size, eps=1e-5, *, stream=None):
    """src/kernel/rms_norm.h:26-34."""
    rc = _lib.load().bz_add_rms_norm(_ptr(input), _ptr(residual), _ptr(weight), bz_dtype(input), num_tokens,
                                     hidden_size, eps, _stream(stream))
    check(rc, "fusedAddRmsNorm")


def silu_and_mul(input, output, num_tokens, inter_size, *, stream=None):
    """src/kernel/activation.h:10-16."""
    rc = _lib.load().bz_silu_and_mul(_ptr(input), _ptr(output), bz_dtype(input), num_tokens, inter_size,
                                     _stream(stream))
    check(rc, "siluAndMul")


def add_residual(input, residual, num_tokens, dim, *, stream=None):
    """src/kernel/add.h:8-14."""
    rc = _lib.load().bz_add_residual(_ptr(input), _ptr(residual), bz_dtype(input), num_tokens, dim, _stream(stream))
    check(rc, "AddKernel")


def embedding(output, token_ids, weight, num_tokens, hidden_size, *, out_loc=None, stream=None):
    """src/kernel/embedding.h:7-36: output[loc] = weight[token_ids[t]]; loc = t or out_loc[t]."""
    rc = _lib.load().bz_embedding(_ptr(output), _ptr(token_ids), _ptr(out_loc) if out_loc is not None else None,
                                  _ptr(weight), bz_dtype(weight), num_tokens, hidden_size, _stream(stream))
    check(rc, "EmbeddingKernel")


def gather_last_token(output, tokens, ragged_indptr, num_tokens, batch_size, hidden_size, *, stream=None):
    """src/kernel/sampler.h:8-16: output[b] = tokens[ragged_indptr[b+1] - 1]."""
    rc = _lib.load().bz_gather_last_token(_ptr(output), _ptr(tokens), _ptr(ragged_indptr), bz_dtype(tokens),
                                          num_tokens, batch_size, hidden_size, _stream(stream))
    check(rc, "GatherLastTokenKernel")


def batch_find_max(output_indices, input, batch_size, length, *, stream=None):
    """src/kernel/sampler.h:18-26: output_indices[b] = argmax(input[b])."""
    rc = _lib.load().bz_batch_find_max(_ptr(output_indices), _ptr(input), bz_dtype(input), batch_size, length,
                                       _stream(stream))
    check(rc, "BatchFindMaxKernel")


def kv_wire_bytes(page_table, num_pages, layer_cnt, wire_dtype=None):
    """Bytes of the migration buffer for num_pages pages of layer_cnt layers."""
    s = page_table.as_struct()
    wd = page_table.kv_dtype if wire_dtype is None else wire_dtype
    return int(_lib.load().bz_kv_wire_bytes(num_pages, layer_cnt, C.byref(s), wd))


def pack_kv_pages(page_table, max_num_pages, page_ids, start_layer, layer_cnt, wire, *, wire_dtype=None,
                  k_scale=None, v_scale=None, stream=None):
    """The messages of MigrationManager::send_multi_layer_fast (src/blitz/migration_manager.h:455-467),
    page by page and layer by layer, concatenated into `wire`.  page_table.base is layer 0 of the pool."""
    s = page_table.as_struct()
    wd = page_table.kv_dtype if wire_dtype is None else wire_dtype
    rc = _lib.load().bz_kv_pages_pack(_ptr(page_table.base), max_num_pages, C.byref(s), _ptr(page_ids),
                                      page_ids.numel(), start_layer, layer_cnt, _ptr(wire), wd, _ptr(k_scale),
                                      _ptr(v_scale), _stream(stream))
    check(rc, "PackKVPages")


def unpack_kv_pages(page_table, max_num_pages, page_ids, start_layer, layer_cnt, wire, *, wire_dtype=None,
                    k_scale=None, v_scale=None, stream=None):
    """The receiving side: chunk i*layer_cnt + l of `wire` goes to page page_ids[i] of layer start_layer + l."""
    s = page_table.as_struct()
    wd = page_table.kv_dtype if wire_dtype is None else wire_dtype
    rc = _lib.load().bz_kv_pages_unpack(_ptr(page_table.base), max_num_pages, C.byref(s), _ptr(page_ids),
                                        page_ids.numel(), start_layer, layer_cnt, _ptr(wire), wd, _ptr(k_scale),
                                        _ptr(v_scale), _stream(stream))
    check(rc, "UnpackKVPages")
