// Drop-in for src/kernel/attention.h: same two entry points, same argument order.
#pragma once

#include "bz_types.h"
#include "flashinfer_types.h"
#include "page.h"

namespace blitz::kernel {

/// src/kernel/attention.h:9-22.  Ragged causal self-attention; q and k are expected rotated already
/// (store_prefill_kv_cache does it together with the page store) unless rope_in_call is set, in which
/// case q and k are rotated in place here first.
template<typename DType, typename IdType>
void batch_prefill_attention(BatchPrefillRaggedHandler<DType, IdType>& handler, DType* q_input, IdType* qo_indptr,
                             DType* k_input, DType* v_input, IdType* kv_indptr, DType* output, uint32_t batch_size,
                             uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_size,
                             bool rope_in_call = false) {
    const AttentionOptions& o = attention_options();
    bz_throw(bz_batch_prefill_ragged(static_cast<bz_prefill_plan_t*>(handler.get()), q_input,
                                     reinterpret_cast<const int32_t*>(qo_indptr), k_input, v_input,
                                     reinterpret_cast<const int32_t*>(kv_indptr), output, bz_dtype<DType>::value,
                                     batch_size, num_qo_heads, num_kv_heads, head_size, /*causal=*/1,
                                     rope_in_call ? BZ_ROPE_FULL : BZ_ROPE_NONE, o.rope_theta, o.sm_scale, o.stream),
             "BatchPrefillWithRaggedKVCache");
}

/// src/kernel/attention.h:24-31.  q, output: [batch, num_qo_heads, head_size].
template<typename DType, typename IdType, typename KVType = DType>
void batch_decode_attention(BlitzBatchDecodeHandler<DType, IdType>& handler, DType* q_input,
                            PageTable<KVType, IdType>& paged_kv, DType* output, const uint32_t num_qo_heads,
                            int rope_mode = -1, const float* k_scale = nullptr, const float* v_scale = nullptr) {
    const AttentionOptions& o = attention_options();
    const bz_paged_kv_t kv = paged_kv.c_view();
    bz_throw(bz_batch_decode(static_cast<bz_decode_plan_t*>(handler.get()), q_input, bz_dtype<DType>::value, &kv, output,
                             bz_dtype<DType>::value, num_qo_heads, rope_mode < 0 ? o.decode_rope_mode : rope_mode,
                             o.rope_theta, o.sm_scale, k_scale, v_scale, nullptr, o.stream),
             "batchDecodeAttention");
}

} // namespace blitz::kernel
