// Drop-in for src/kernel/page.h of the BlitzScale worker: the per-batch page table and the two
// KV-page writers, over the C ABI of libbz_hip.so.
#pragma once

#include <cstddef>
#include <cstdint>
#include <vector>

#include "bz_types.h"

namespace blitz::kernel {

/// Per-batch CSR page table plus the base pointers of one layer plane of the pool
/// (same members as the reference struct, src/kernel/page.h:12-64, plus the in-page layout).
/// Element address: page*stride_page + slot*stride_n + head*stride_h + d from k_data / v_data.
template<typename DType, typename IdType>
struct PageTable {
    // host copy, maintained by the cache manager
    std::vector<IdType> indices;
    std::vector<IdType> indptr;
    std::vector<IdType> last_page_len;
    uint32_t batch_size;

    const uint32_t page_size;
    const uint32_t num_heads;
    const uint32_t head_size;

    const size_t stride_page; // 2 * num_heads * page_size * head_size: K half then V half
    const size_t stride_n;    // between consecutive slots of one head
    const size_t stride_h;    // between heads
    const int layout;         // BZ_LAYOUT_HND (default) or BZ_LAYOUT_NHD (the reference's order)

    // pinned host blob [indices | indptr | last_page_len]
    IdType* indices_h = nullptr;
    IdType* indptr_h = nullptr;
    IdType* last_page_len_h = nullptr;

    // one layer plane: v_data = k_data + num_heads * page_size * head_size
    DType* k_data;
    DType* v_data;
    // device copy of the table, set by the caller right before a step (src/blitz/stub.h:1310-1313)
    IdType* indices_d = nullptr;
    IdType* indptr_d = nullptr;
    IdType* last_page_len_d = nullptr;
    // optional device counter: the table describes the batch this many decode steps ahead of the present
    // (pages of the tokens to come already listed); nullptr = the table is the present
    IdType* steps_ahead_d = nullptr;
    // RoPE base / placement and stream of the page writes made through this table: the model's own
    // (e.g. &decode_handler.options); nullptr = those of the handler that planned last on this thread, and
    // the process-wide default before any plan
    const AttentionOptions* options = nullptr;
    const AttentionOptions& opts() const {
        if (options) return *options;
        return planned_options().valid ? planned_options().value : attention_options();
    }

    PageTable(uint32_t batch_size_, uint32_t page_size_, uint32_t num_heads_, uint32_t head_size_, DType* base_ptr,
              int layout_ = BZ_LAYOUT_HND) :
        batch_size(batch_size_),
        page_size(page_size_),
        num_heads(num_heads_),
        head_size(head_size_),
        stride_page((size_t)2 * num_heads_ * page_size_ * head_size_),
        stride_n(layout_ == BZ_LAYOUT_HND ? (size_t)head_size_ : (size_t)num_heads_ * head_size_),
        stride_h(layout_ == BZ_LAYOUT_HND ? (size_t)page_size_ * head_size_ : (size_t)head_size_),
        layout(layout_),
        k_data(base_ptr),
        v_data(base_ptr + (size_t)num_heads_ * page_size_ * head_size_) {}

    /// plain-C image handed to the library
    bz_paged_kv_t c_view() const {
        bz_paged_kv_t kv;
        kv.k_data = k_data; kv.v_data = v_data;
        kv.indices = reinterpret_cast<const int32_t*>(indices_d);
        kv.indptr = reinterpret_cast<const int32_t*>(indptr_d);
        kv.last_page_len = reinterpret_cast<const int32_t*>(last_page_len_d);
        kv.batch_size = batch_size; kv.page_size = page_size; kv.num_kv_heads = num_heads; kv.head_dim = head_size;
        kv.stride_page = stride_page; kv.stride_n = stride_n; kv.stride_h = stride_h;
        kv.kv_dtype = bz_dtype<DType>::value; kv.reserved = 0;
        kv.steps_ahead = reinterpret_cast<const int32_t*>(steps_ahead_d);
        return kv;
    }
};

/// Token t of request b goes to page indices[indptr[b] + t/P], slot t%P (src/kernel/page.cu:21-62).
/// num_tokens: rows of k_data / v_data.  q_inout (optional, [N, num_qo_heads, D]): the fused RoPE of the
/// prefill path -- K is rotated on its way into the pages and q and the caller's k rows are rotated in
/// place by the same angles, so that batch_prefill_attention runs with BZ_ROPE_NONE afterwards.
/// rotate: 1 / 0 force K rotation on / off, 2 = rotate K into the pages AND in place in the caller's rows
/// (q is then left to batch_prefill_attention with BZ_ROPE_Q_ONLY), < 0 = on when q_inout is given, else
/// opts().store_rotates_k.  options: whose RoPE base and stream to use (a layer passes its handler's, so that
/// the pages and the attention call cannot disagree); nullptr = page_table.opts().
template<typename DType, typename IdType, typename SrcType = DType>
void store_prefill_kv_cache(PageTable<DType, IdType>& page_table, SrcType* k_data, SrcType* v_data,
                            IdType* ragged_indptr, uint32_t num_tokens, SrcType* q_inout = nullptr,
                            uint32_t num_qo_heads = 0, const float* k_scale = nullptr,
                            const float* v_scale = nullptr, int rotate = -1, const AttentionOptions* options = nullptr) {
    static_assert(sizeof(IdType) == 4, "page tables are int32");
    const AttentionOptions& o = options ? *options : page_table.opts();
    const bz_paged_kv_t kv = page_table.c_view();
    const int rot = rotate < 0 ? ((q_inout != nullptr || o.store_rotates_k) ? 1 : 0) : rotate;
    bz_throw(bz_store_prefill_kv(&kv, k_data, v_data, bz_dtype<SrcType>::value,
                                 reinterpret_cast<const int32_t*>(ragged_indptr), num_tokens, q_inout, num_qo_heads,
                                 rot, o.rope_theta, k_scale, v_scale, o.stream),
             "AppendPagedKVCache");
}

/// src/kernel/page.h:66-67, the reference's own four arguments (called at src/layer/attn.h:188-193 right
/// after batch_prefill_attention).  The token count is read on the device from ragged_indptr[batch_size],
/// like the reference's launch, which is shaped by page size and batch alone (page.cu:84-89).  K is stored
/// as it is found unless opts().store_rotates_k says otherwise: under the reference's call order the
/// attention call has rotated it already.
template<typename DType, typename IdType, typename SrcType = DType>
void store_prefill_kv_cache(PageTable<DType, IdType>& page_table, SrcType* k_data, SrcType* v_data,
                            IdType* ragged_indptr) {
    store_prefill_kv_cache(page_table, k_data, v_data, ragged_indptr, BZ_NUM_TOKENS_FROM_INDPTR);
}

/// src/kernel/page.h:69-70.  One new row per sequence at position seq_len-1.  With the reference's three
/// arguments the new K row is rotated on its way in (opts().append_rotates_k) and nothing else is touched;
/// q_inout (optional, [B, num_qo_heads, D]) is the fused form: q is rotated in place as well, and
/// batch_decode_attention runs with BZ_ROPE_NONE afterwards.
/// rotate: 1 / 0 force K rotation on / off, < 0 = on when q_inout is given, else opts().append_rotates_k.
/// options: as for store_prefill_kv_cache.
template<typename DType, typename IdType, typename SrcType = DType>
void append_decode_kv_cache(PageTable<DType, IdType>& page_table, SrcType* k_data, SrcType* v_data,
                            SrcType* q_inout = nullptr, uint32_t num_qo_heads = 0, const float* k_scale = nullptr,
                            const float* v_scale = nullptr, int rotate = -1, const AttentionOptions* options = nullptr) {
    static_assert(sizeof(IdType) == 4, "page tables are int32");
    const AttentionOptions& o = options ? *options : page_table.opts();
    const bz_paged_kv_t kv = page_table.c_view();
    const bool rot = rotate < 0 ? (q_inout != nullptr || o.append_rotates_k) : rotate != 0;
    bz_throw(bz_append_decode_kv(&kv, k_data, v_data, bz_dtype<SrcType>::value, q_inout, num_qo_heads, rot ? 1 : 0,
                                 o.rope_theta, k_scale, v_scale, o.stream),
             "AppendPagedKVCacheDecode");
}

/// The cached K rows of every sequence of the table rotated in place at their positions (inverse: the rotation
/// taken off again): converts a cache that holds K as the projection left it -- the reference's convention, under
/// which attention_decode.cu:35 rotates every cached row at every step -- to the rotated-K cache the decode calls
/// here expect, once, at the speed of a copy.  No counterpart in the reference.
template<typename DType, typename IdType>
void rope_cached_k(PageTable<DType, IdType>& page_table, bool inverse = false, const AttentionOptions* options = nullptr) {
    const AttentionOptions& o = options ? *options : page_table.opts();
    const bz_paged_kv_t kv = page_table.c_view();
    bz_throw(bz_rope_cached_k(&kv, o.rope_theta, inverse ? 1 : 0, o.stream), "ropeCachedK");
}

/// declared and never defined in the reference (src/kernel/page.h:72-73); here it is the token count
template<typename DType, typename IdType>
uint32_t cal_total_num_rows(const PageTable<DType, IdType>& page_table) {
    uint32_t rows = 0;
    for (uint32_t b = 0; b < page_table.batch_size; ++b) {
        const IdType n = page_table.indptr[b + 1] - page_table.indptr[b];
        if (n > 0) rows += (uint32_t)(n - 1) * page_table.page_size + (uint32_t)page_table.last_page_len[b];
    }
    return rows;
}

} // namespace blitz::kernel
