// Drop-in for src/kernel/attention.h: same two entry points, same argument order.
#pragma once

#include "bz_types.h"
#include "flashinfer_types.h"
#include "page.h"

namespace blitz::kernel {

/// src/kernel/attention.h:9-22.  Ragged causal attention over q [Nq,Hq,D], k,v [Nkv,Hkv,D]: self-attention when
/// qo_indptr and kv_indptr are the same array (the reference's only use); with two arrays a request brings q rows
/// for its last tokens only and K/V rows for all of them (what plan() was given must match).
/// rope_mode < 0 takes handler.options.prefill_rope_mode, whose default BZ_ROPE_FULL is the reference's
/// kRoPELlama (attention_prefill.cu:38): q rows are rotated by their position inside the request in registers (in
/// place only when the float workspace has no room for the angle table), k rows IN PLACE in the caller's buffer,
/// before the contraction; k then holds what the cache must hold, and
/// store_prefill_kv_cache that follows (src/layer/attn.h:188-193) must not rotate it again (its default).
/// BZ_ROPE_NONE: q and k are used as they are (they were rotated while the pages were written).
template<typename DType, typename IdType>
void batch_prefill_attention(BatchPrefillRaggedHandler<DType, IdType>& handler, DType* q_input, IdType* qo_indptr,
                             DType* k_input, DType* v_input, IdType* kv_indptr, DType* output, uint32_t batch_size,
                             uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_size, int rope_mode = -1) {
    const AttentionOptions& o = handler.options;
    bz_throw(bz_batch_prefill_ragged(static_cast<bz_prefill_plan_t*>(handler.get()), q_input,
                                     reinterpret_cast<const int32_t*>(qo_indptr), k_input, v_input,
                                     reinterpret_cast<const int32_t*>(kv_indptr), output, bz_dtype<DType>::value,
                                     batch_size, num_qo_heads, num_kv_heads, head_size, /*causal=*/1,
                                     rope_mode < 0 ? o.prefill_rope_mode : rope_mode, o.rope_theta, o.sm_scale, o.stream),
             "BatchPrefillWithRaggedKVCache");
}

/// src/kernel/attention.h:24-31.  q, output: [batch, num_qo_heads, head_size].  rope_mode < 0 takes
/// handler.options.decode_rope_mode (default BZ_ROPE_Q_ONLY: q is rotated at position seq_len-1 inside the
/// kernel, the caller's q stays as it is; cached K is rotated already).
template<typename DType, typename IdType, typename KVType = DType>
void batch_decode_attention(BlitzBatchDecodeHandler<DType, IdType>& handler, DType* q_input,
                            PageTable<KVType, IdType>& paged_kv, DType* output, const uint32_t num_qo_heads,
                            int rope_mode = -1, const float* k_scale = nullptr, const float* v_scale = nullptr) {
    const AttentionOptions& o = handler.options;
    const bz_paged_kv_t kv = paged_kv.c_view();
    bz_throw(bz_batch_decode(static_cast<bz_decode_plan_t*>(handler.get()), q_input, bz_dtype<DType>::value, &kv, output,
                             bz_dtype<DType>::value, num_qo_heads, rope_mode < 0 ? o.decode_rope_mode : rope_mode,
                             o.rope_theta, o.sm_scale, k_scale, v_scale, nullptr, o.stream),
             "batchDecodeAttention");
}

/// append_decode_kv_cache followed by batch_decode_attention (src/layer/attn.h:196-203) as ONE call, two
/// launches instead of three (no counterpart in the reference): the new K row (rotated when
/// handler.options.append_rotates_k) and V row go into the cache, q is rotated inside the kernels, and q, k, v
/// stay as the projection left them.  Same cache bits as the two calls, same result to rounding.
template<typename DType, typename IdType, typename KVType = DType>
void decode_attention_step(BlitzBatchDecodeHandler<DType, IdType>& handler, DType* q_input, DType* k_new, DType* v_new,
                           PageTable<KVType, IdType>& paged_kv, DType* output, const uint32_t num_qo_heads,
                           const float* k_scale = nullptr, const float* v_scale = nullptr) {
    const AttentionOptions& o = handler.options;
    const bz_paged_kv_t kv = paged_kv.c_view();
    bz_throw(bz_decode_step(static_cast<bz_decode_plan_t*>(handler.get()), q_input, bz_dtype<DType>::value, k_new, v_new,
                            &kv, output, bz_dtype<DType>::value, num_qo_heads, o.append_rotates_k ? 1 : 0, o.rope_theta,
                            o.sm_scale, k_scale, v_scale, nullptr, o.stream),
             "batchDecodeAttention");
}

} // namespace blitz::kernel
