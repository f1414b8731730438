// Shared device/host helpers for the gfx950 kernels: storage-type traits, 16-byte vector
// access, wave64 reductions.  CDNA4 only: wavefront size is 64 everywhere in this library.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "../../include/bz_hip.h"

#define BZ_CHECK_HIP(expr)                         \
    do {                                           \
        hipError_t _e = (expr);                    \
        if (_e != hipSuccess) return (int)_e;      \
    } while (0)

#define BZ_LAUNCH_CHECK()                          \
    do {                                           \
        hipError_t _e = hipGetLastError();         \
        if (_e != hipSuccess) return (int)_e;      \
    } while (0)

namespace bz {

constexpr int kWave = 64;

struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };
struct e4m3_t { uint8_t bits; };

// ---- scalar conversions (device) -------------------------------------------------------
__device__ __forceinline__ float to_f32(f16_t v) {
    return __half2float(__ushort_as_half(v.bits));
}
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }
__device__ __forceinline__ float to_f32(float v) { return v; }

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __half_as_ushort(__float2half_rn(f)); }
// fp32 -> bf16, round to nearest even, on the conversion unit of gfx950 (v_cvt_pk_bf16_f32: two values per
// instruction; the bit-twiddled form costs six vector instructions per value)
typedef __attribute__((ext_vector_type(2))) __bf16 bz_bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float bz_f32x2_t;
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
    const bz_f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bz_bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(f32x2_to_bf16x2_bits(f, 0.f) & 0xffffu); }

// One rotate-half pair: (x, y) -> (x c - y s, y c + x s).  Every product and sum is rounded on its own
// (no fused multiply-add), so that all kernels of the library that rotate the same row get the same
// bits, and so does a scalar restatement compiled without contraction.
__device__ __forceinline__ void rope_pair(float x, float y, float c, float s, float& xr, float& yr) {
#pragma clang fp contract(off)
    const float xc = x * c, ys = y * s, yc = y * c, xs = x * s;
    xr = xc - ys;
    yr = yc + xs;
}

// Reductions over the lanes l, l^16 (and l^32) of a wave with the gfx950 lane-swap instructions: the
// partner's value arrives through the vector ALU instead of an LDS round trip (ds_bpermute).  With the
// same value in both operands v_permlane16_swap leaves rows {0,0,2,2} in the first result and rows
// {1,1,3,3} in the second, v_permlane32_swap the lower half twice and the upper half twice.
__device__ __forceinline__ float lane_max_xor16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane_max_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane_sum_xor16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float lane_sum_xor32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <typename T> struct StoreCvt;
template <> struct StoreCvt<f16_t> {
    __device__ static __forceinline__ f16_t from(float f) { return f16_t{f32_to_f16_bits(f)}; }
};
template <> struct StoreCvt<bf16_t> {
    __device__ static __forceinline__ bf16_t from(float f) { return bf16_t{f32_to_bf16_bits(f)}; }
};
template <> struct StoreCvt<float> {
    __device__ static __forceinline__ float from(float f) { return f; }
};

// OCP e4m3fn -> fp32 for two packed bytes (gfx950 conversion unit is OCP, not FNUZ)
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float* out) {
    auto lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
    auto hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}
// fp32 -> OCP e4m3fn, round-to-nearest-even, saturating at +-448
__device__ __forceinline__ uint8_t f32_to_e4m3_bits(float f) {
    f = fminf(fmaxf(f, -448.0f), 448.0f);
    uint32_t r = __builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false);
    return (uint8_t)(r & 0xffu);
}

// ---- 8-element vectors ------------------------------------------------------------------
// Vec8<T>: eight consecutive elements of a row.  16 bytes for f16/bf16, 8 bytes for e4m3.
template <typename T> struct Vec8;

template <> struct Vec8<f16_t> {
    uint4 raw;
    __device__ __forceinline__ void load(const void* p) { raw = *reinterpret_cast<const uint4*>(p); }
    __device__ __forceinline__ void load_nt(const void* p) { // for data that is read once
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        raw = make_uint4(v.x, v.y, v.z, v.w);
    }
    __device__ __forceinline__ void store(void* p) const { *reinterpret_cast<uint4*>(p) = raw; }
    __device__ __forceinline__ void store_nt(void* p) const { // for data that is not read again soon
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = {raw.x, raw.y, raw.z, raw.w};
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
    }
    __device__ __forceinline__ void to_float(float* f) const {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __half2float(__ushort_as_half((uint16_t)(w[i] & 0xffffu)));
            f[2 * i + 1] = __half2float(__ushort_as_half((uint16_t)(w[i] >> 16)));
        }
    }
    __device__ __forceinline__ void from_float(const float* f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = (uint32_t)f32_to_f16_bits(f[2 * i]) | ((uint32_t)f32_to_f16_bits(f[2 * i + 1]) << 16);
        raw = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

template <> struct Vec8<bf16_t> {
    uint4 raw;
    __device__ __forceinline__ void load(const void* p) { raw = *reinterpret_cast<const uint4*>(p); }
    __device__ __forceinline__ void load_nt(const void* p) { // for data that is read once
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
        raw = make_uint4(v.x, v.y, v.z, v.w);
    }
    __device__ __forceinline__ void store(void* p) const { *reinterpret_cast<uint4*>(p) = raw; }
    __device__ __forceinline__ void store_nt(void* p) const { // for data that is not read again soon
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = {raw.x, raw.y, raw.z, raw.w};
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
    }
    __device__ __forceinline__ void to_float(float* f) const {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(w[i] << 16);
            f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    }
    __device__ __forceinline__ void from_float(const float* f) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = f32x2_to_bf16x2_bits(f[2 * i], f[2 * i + 1]);
        raw = make_uint4(w[0], w[1], w[2], w[3]);
    }
};

template <> struct Vec8<e4m3_t> {
    uint2 raw;
    __device__ __forceinline__ void load(const void* p) { raw = *reinterpret_cast<const uint2*>(p); }
    __device__ __forceinline__ void load_nt(const void* p) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
        raw = make_uint2(v.x, v.y);
    }
    __device__ __forceinline__ void store(void* p) const { *reinterpret_cast<uint2*>(p) = raw; }
    __device__ __forceinline__ void store_nt(void* p) const {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        const u32x2 v = {raw.x, raw.y};
        __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p));
    }
    __device__ __forceinline__ void to_float(float* f) const {
        e4m3x4_to_f32(raw.x, f);
        e4m3x4_to_f32(raw.y, f + 4);
    }
    __device__ __forceinline__ void from_float(const float* f) {
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int i = 0; i < 8; ++i) w[i / 4] |= (uint32_t)f32_to_e4m3_bits(f[i]) << (8 * (i % 4));
        raw = make_uint2(w[0], w[1]);
    }
};

template <> struct Vec8<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const void* p) {
        a = reinterpret_cast<const float4*>(p)[0];
        b = reinterpret_cast<const float4*>(p)[1];
    }
    __device__ __forceinline__ void store(void* p) const {
        reinterpret_cast<float4*>(p)[0] = a;
        reinterpret_cast<float4*>(p)[1] = b;
    }
    __device__ __forceinline__ void to_float(float* f) const {
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
    __device__ __forceinline__ void from_float(const float* f) {
        a = make_float4(f[0], f[1], f[2], f[3]);
        b = make_float4(f[4], f[5], f[6], f[7]);
    }
};

template <typename T> __device__ __forceinline__ constexpr size_t elem_size() { return sizeof(T); }

// ---- wave64 reductions -------------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Llama rotate-half frequencies, f_i = theta^(-2i/D), evaluated in double on the host and rounded
// to fp32 so that host checker and device use bit-identical angles pos*f_i.
struct RopeFreqs {
    float f[64]; // head_dim <= 128
};

inline RopeFreqs make_rope_freqs(int D, float theta) {
    RopeFreqs r;
    for (int i = 0; i < 64; ++i) r.f[i] = 0.f;
    for (int i = 0; i < D / 2 && i < 64; ++i) r.f[i] = (float)pow((double)theta, -2.0 * (double)i / (double)D);
    return r;
}

inline size_t dtype_bytes(int dt) { return dt == BZ_F32 ? 4 : (dt == BZ_E4M3 ? 1 : 2); }

} // namespace bz
