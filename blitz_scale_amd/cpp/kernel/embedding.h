// Drop-in for src/kernel/embedding.h.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

/// output[t] = embed_tokens_weight[token_ids[t]] (src/kernel/embedding.h:7-14, embedding.cu:48-66).
template<typename DType>
void embedding(DType* output, const uint32_t* token_ids, const DType* embed_tokens_weight, const uint32_t num_tokens,
               const uint32_t hidden_size, void* stream = kStreamFromOptions) {
    bz_throw(bz_embedding(output, token_ids, nullptr, embed_tokens_weight, bz_dtype<DType>::value, num_tokens,
                          hidden_size, resolve_stream(stream)),
             "EmbeddingKernel");
}

/// output[out_loc[t]] = embed_tokens_weight[token_ids[t]]: the tensor-parallel variant that scatters the
/// locally held rows into a zeroed buffer before the all-reduce (src/kernel/embedding.h:16-36,
/// embedding.cu:68-89).
template<typename DType, typename IdType>
void embedding(DType* output, const uint32_t* token_ids, const IdType* out_loc, const DType* embed_tokens_weight,
               const uint32_t num_tokens, const uint32_t hidden_size, void* stream = kStreamFromOptions) {
    static_assert(sizeof(IdType) == 4, "page and row ids are 32-bit, as in the reference's instantiation");
    bz_throw(bz_embedding(output, token_ids, reinterpret_cast<const int32_t*>(out_loc), embed_tokens_weight,
                          bz_dtype<DType>::value, num_tokens, hidden_size, resolve_stream(stream)),
             "EmbeddingKernel");
}

} // namespace blitz::kernel
