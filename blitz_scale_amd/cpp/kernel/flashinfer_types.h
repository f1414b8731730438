// Drop-in for src/kernel/flashinfer_types.h: the two handler classes keep their names and plan()
// signatures; behind them sit the library's own planners instead of FlashInfer handlers.
#pragma once

#include "bz_types.h"

namespace blitz::kernel {

inline void* create_flashinfer_prefill_handler() { return bz_prefill_plan_create(); }
inline void* create_flashinfer_decode_handler() { return bz_decode_plan_create(); }

template<typename DType, typename IdType>
class BatchPrefillRaggedHandler {
  public:
    /// src/kernel/flashinfer_types.h:15-27: host scheduling from the host indptr arrays
    void plan(void* float_buffer, size_t float_buffer_size, void* int_buffer, size_t int_buffer_size,
              IdType* qo_indptr_h, IdType* kv_indptr_h, uint32_t batch_size, uint32_t num_qo_heads,
              uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size) {
        bz_throw(bz_prefill_plan(static_cast<bz_prefill_plan_t*>(handler_), float_buffer, float_buffer_size, int_buffer,
                                 int_buffer_size, reinterpret_cast<const int32_t*>(qo_indptr_h),
                                 reinterpret_cast<const int32_t*>(kv_indptr_h), batch_size, num_qo_heads, num_kv_heads,
                                 head_dim, page_size, options.stream),
                 "Handler plan:");
        bz_throw(bz_prefill_plan_set_bf16_mode(static_cast<bz_prefill_plan_t*>(handler_), options.prefill_bf16_mode),
                 "Handler plan:");
        note_planned_options(options);
    }
    BatchPrefillRaggedHandler(void* handler_ptr = nullptr) : handler_(handler_ptr) {}
    void* get() noexcept { return handler_; }
    bool empty() noexcept { return handler_ == nullptr; }

    /// RoPE base, softmax scale, RoPE placement and stream of the calls made through this handler
    /// (a copy of the process-wide default at construction; set per model / per thread)
    AttentionOptions options = attention_options();

  private:
    void* handler_;
};

template<typename DType, typename IdType>
class BlitzBatchDecodeHandler {
  public:
    /// src/kernel/flashinfer_types.h:46-58: split-K scheduling from the host indptr / last_page_len
    void plan(void* float_buffer, size_t float_buffer_size, void* int_buffer, size_t int_buffer_size,
              IdType* qo_indptr_h, IdType* last_page_len_h, uint32_t batch_size, uint32_t num_qo_heads,
              uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size) {
        const AttentionOptions& o = options;
        bz_throw(bz_decode_plan(static_cast<bz_decode_plan_t*>(handler_), float_buffer, float_buffer_size, int_buffer,
                                int_buffer_size, reinterpret_cast<const int32_t*>(qo_indptr_h),
                                reinterpret_cast<const int32_t*>(last_page_len_h), batch_size, num_qo_heads,
                                num_kv_heads, head_dim, page_size, o.split_tokens, o.stream),
                 "Handler plan:");
        note_planned_options(options);
    }
    BlitzBatchDecodeHandler(void* handler_ptr = nullptr) : handler_(handler_ptr) {}
    void* get() noexcept { return handler_; }
    bool empty() noexcept { return handler_ == nullptr; }

    /// as for the prefill handler: this handler's own copy of the options
    AttentionOptions options = attention_options();

  private:
    void* handler_;
};

} // namespace blitz::kernel
