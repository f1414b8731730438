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

/// Parameters the reference never passes (FlashInfer defaults apply there): RoPE base, softmax
/// scale, RoPE handling and the stream.  One process-wide default keeps the reference's call
/// signatures unchanged; a serving engine sets it once from the model config.
struct AttentionOptions {
    float rope_theta = 1e4f;          // Llama-2; Llama-3 uses 5e5
    float sm_scale = 0.f;             // <= 0: 1/sqrt(head_dim)
    int decode_rope_mode = BZ_ROPE_Q_ONLY;  // K is cached rotated (append/store rotate it)
    bool rotate_k_on_write = true;    // append_decode_kv_cache / store_prefill_kv_cache rotate K
    uint32_t split_tokens = 0;        // 0: library default (2048)
    void* stream = nullptr;           // legacy default stream, as the reference
};
inline AttentionOptions& attention_options() {
    static AttentionOptions opts;
    return opts;
}

} // namespace blitz::kernel
