// Drop-in for src/kernel/sampler.h.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

/// output[b] = tokens[ragged_indptr[b+1] - 1], the whole hidden row (src/kernel/sampler.h:8-16; the
/// reference's kernel writes every lane's slice to the start of the row, sampler.cu:21-24).
template<typename DType, typename IdType>
void gather_last_token(DType* output, const DType* tokens, const IdType* ragged_indptr, const uint32_t num_tokens,
                       const uint32_t batch_size, const uint32_t hidden_size, void* stream = kStreamFromOptions) {
    static_assert(sizeof(IdType) == 4, "row ids are 32-bit, as in the reference's instantiation");
    bz_throw(bz_gather_last_token(output, tokens, reinterpret_cast<const int32_t*>(ragged_indptr), bz_dtype<DType>::value,
                                  num_tokens, batch_size, hidden_size, resolve_stream(stream)),
             "GatherLastTokenKernel");
}

/// output_indices[b] = argmax over input[b][0..length) (src/kernel/sampler.h:18-26): the smallest index
/// of the largest value.
template<typename DType>
void batch_find_max(uint32_t* output_indices, const DType* input, const uint32_t batch_size, const uint32_t length,
                    void* stream = kStreamFromOptions) {
    bz_throw(bz_batch_find_max(output_indices, input, bz_dtype<DType>::value, batch_size, length,
                               resolve_stream(stream)),
             "BatchFindMaxKernel");
}

} // namespace blitz::kernel
