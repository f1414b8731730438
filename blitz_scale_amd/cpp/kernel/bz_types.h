// Element-type tags and the error convention shared by the C++ drop-in headers.
// The reference wrappers throw std::runtime_error("<name> error: <text>") on a non-zero status
// (e.g. src/kernel/attention_decode.cu:37-39); bz_throw does the same for the C ABI's codes.
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "bz_hip.h"

namespace blitz::kernel {

struct e4m3_storage { uint8_t bits; }; // OCP e4m3fn byte of an fp8 KV pool

template<typename T> struct bz_dtype;
template<> struct bz_dtype<__half> { static constexpr int value = BZ_F16; };
template<> struct bz_dtype<__hip_bfloat16> { static constexpr int value = BZ_BF16; };
template<> struct bz_dtype<e4m3_storage> { static constexpr int value = BZ_E4M3; };
template<> struct bz_dtype<float> { static constexpr int value = BZ_F32; };

inline void bz_throw(int status, const char* what) {
    if (status != 0) throw std::runtime_error(std::string(what) + " error: " + bz_error_string(status));
}

/// Parameters the reference never passes (FlashInfer defaults apply there): RoPE base, softmax scale,
/// where RoPE is applied, and the stream.  They travel with the objects the reference's calls already
/// take -- every handler (BatchPrefillRaggedHandler, BlitzBatchDecodeHandler) holds its own copy and a
/// PageTable may point at one -- so two models, or two host threads on two streams, do not share them;
/// attention_options() is only the process-wide default a new handler starts from.
///
/// The RoPE defaults give the reference's kRoPELlama results (attention_prefill.cu:38,
/// attention_decode.cu:35) under the reference's own call order (src/layer/attn.h:173-204) with K cached
/// rotated:
///   prefill: batch_prefill_attention rotates q and k (in place, in the caller's activation buffers),
///            store_prefill_kv_cache then stores k as it finds it;
///   decode : append_decode_kv_cache rotates the new K row on its way into the cache,
///            batch_decode_attention rotates q inside the kernel and reads cached K as stored.
struct AttentionOptions {
    float rope_theta = 1e4f;                // Llama-2; Llama-3 uses 5e5
    float sm_scale = 0.f;                   // <= 0: 1/sqrt(head_dim)
    int prefill_rope_mode = BZ_ROPE_FULL;   // batch_prefill_attention: rotate q and k rows before the contraction
    bool store_rotates_k = false;           // store_prefill_kv_cache: k was rotated by the attention call before it
    bool append_rotates_k = true;           // append_decode_kv_cache rotates the new K row
    int decode_rope_mode = BZ_ROPE_Q_ONLY;  // batch_decode_attention: rotate q only, cached K is rotated
    uint32_t split_tokens = 0;              // 0: library default (2048)
    int prefill_bf16_mode = BZ_PREFILL_BF16_WIDEN_V; // bf16 prefill: second product in f16 with V widened (exact for
                                            // |v| in f16's range), or BZ_PREFILL_BF16_HEAD_TAIL for any range of V
    void* stream = nullptr;                 // hipStream_t; nullptr = the legacy default stream the reference uses
};
inline AttentionOptions& attention_options() {
    static AttentionOptions opts;
    return opts;
}

/// The options of the handler that planned last on this host thread (a copy, taken by plan()).  The page
/// writes of the reference's calls take a PageTable and no handler; a table that points at no options of its own
/// falls back to these, so that an engine which sets the RoPE base on its handlers only -- and builds a new
/// PageTable per batch -- still gets the pages written with the base its attention calls use.  (Per thread: two
/// models on two threads do not see each other; two models on one thread each plan before their layers run.)
struct PlannedOptions {
    AttentionOptions value;
    bool valid = false;
};
inline PlannedOptions& planned_options() {
    thread_local PlannedOptions p;
    return p;
}
inline void note_planned_options(const AttentionOptions& o) {
    planned_options().value = o;
    planned_options().valid = true;
}

/// "no stream argument given": the element-wise wrappers then launch on attention_options().stream
inline void* const kStreamFromOptions = reinterpret_cast<void*>(~static_cast<uintptr_t>(0));
inline void* resolve_stream(void* stream) { return stream == kStreamFromOptions ? attention_options().stream : stream; }

} // namespace blitz::kernel
