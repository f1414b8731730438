// Drop-in for src/kernel/add.h.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

/// residual += input with one rounding per element (src/kernel/add.h:8-14, add.cu:29-32).
template<typename DType>
void add_residual(DType* input, DType* residual, uint32_t num_tokens, uint32_t dim,
                  void* stream = kStreamFromOptions) {
    bz_throw(bz_add_residual(input, residual, bz_dtype<DType>::value, num_tokens, dim, resolve_stream(stream)),
             "AddKernel");
}

} // namespace blitz::kernel
