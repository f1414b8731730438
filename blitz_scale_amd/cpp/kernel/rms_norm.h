// Drop-in for src/kernel/rms_norm.h.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

/// output = input * rsqrt(mean(input^2) + eps) * weight, row-wise; input may alias output
/// (src/kernel/rms_norm.h:11-19, called in place at src/model/llama.h:389-391).
template<typename DType>
void rms_norm(DType* input, DType* weight, DType* output, uint32_t num_tokens, uint32_t hidden_size, float eps = 1e-5,
              void* stream = kStreamFromOptions) {
    bz_throw(bz_rms_norm(input, weight, output, bz_dtype<DType>::value, num_tokens, hidden_size, eps,
                         resolve_stream(stream)),
             "rmsNorm");
}

/// residual += input; input = rms_norm(residual) * weight (src/kernel/rms_norm.h:26-34).
template<typename DType>
void add_rms_norm(DType* input, DType* residual, DType* weight, uint32_t num_tokens, uint32_t hidden_size,
                  float eps = 1e-5, void* stream = kStreamFromOptions) {
    bz_throw(bz_add_rms_norm(input, residual, weight, bz_dtype<DType>::value, num_tokens, hidden_size, eps,
                             resolve_stream(stream)),
             "fusedAddRmsNorm");
}

} // namespace blitz::kernel
