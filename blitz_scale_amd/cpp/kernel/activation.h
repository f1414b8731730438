// Drop-in for src/kernel/activation.h.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

/// output[n, i] = silu(input[n, i]) * input[n, inter_size + i]; gate is the first half
/// (src/kernel/activation.h:7-16).  Unlike the reference wrapper (activation.cu:18-23) a launch
/// failure is reported.
template<typename DType>
void silu_and_mul(DType* input, DType* output, uint32_t num_tokens, uint32_t inter_size,
                  void* stream = kStreamFromOptions) {
    bz_throw(bz_silu_and_mul(input, output, bz_dtype<DType>::value, num_tokens, inter_size, resolve_stream(stream)),
             "siluAndMul");
}

} // namespace blitz::kernel
