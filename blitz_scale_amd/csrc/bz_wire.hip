// KV page wire format for migration between instances: gather the (page, layer) chunks of a batch
// from the pool into one contiguous buffer and scatter them back on the other side.  Replaces the
// per-message addressing of src/blitz/migration_manager.h:86-92 (get_page_ptr) and the send order of
// :455-467 (request by request, prompt block by prompt block, layer by layer; the receive loops
// mirror it): chunk c = i*layer_cnt + l of the buffer is page page_ids[i] of layer start_layer + l,
// stride_page elements long, i.e. the buffer is the concatenation of the reference's messages.  One
// large transfer then replaces one send per (page, layer).  With an e4m3 wire and a 16-bit pool the
// elements travel as x/scale in e4m3 (half the bytes) and come back as e4m3*scale.
//
// HBM-bound copies: every lane moves four 8-element vectors, all four loads in flight before the
// first store.
#include <cstdio>

#include "bz_common.hpp"

namespace bz {

typedef __attribute__((ext_vector_type(4))) uint32_t wire_u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t wire_u32x2;
// Streaming (non-temporal) accesses: every byte is touched once, so nothing is worth keeping in the
// caches (measured: pack 4.9 -> 5.5 TB/s).
template <typename T> __device__ __forceinline__ void wire_load(Vec8<T>& v, const void* p) {
    if constexpr (sizeof(v.raw) == 16) {
        const wire_u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const wire_u32x4*>(p));
        v.raw = make_uint4(r.x, r.y, r.z, r.w);
    } else {
        const wire_u32x2 r = __builtin_nontemporal_load(reinterpret_cast<const wire_u32x2*>(p));
        v.raw = make_uint2(r.x, r.y);
    }
}
template <typename T> __device__ __forceinline__ void wire_store(const Vec8<T>& v, void* p) {
    if constexpr (sizeof(v.raw) == 16) {
        const wire_u32x4 r = {v.raw.x, v.raw.y, v.raw.z, v.raw.w};
        __builtin_nontemporal_store(r, reinterpret_cast<wire_u32x4*>(p));
    } else {
        const wire_u32x2 r = {v.raw.x, v.raw.y};
        __builtin_nontemporal_store(r, reinterpret_cast<wire_u32x2*>(p));
    }
}

constexpr int kWirePer = 4; // vectors per lane

struct WireArgs {
    char* pool;            // base of the whole pool (layer 0)
    char* wire;
    const int32_t* page_ids;
    const float* k_scale;  // [layer_cnt][num_kv_heads] or null
    const float* v_scale;
    uint64_t max_pages;
    uint64_t stride_page;  // elements
    uint64_t stride_h;     // elements
    uint64_t total_vecs;   // num_pages * layer_cnt * stride_page / 8
    uint32_t vecs_per_chunk;
    uint32_t num_kv_heads;
    uint32_t start_layer, layer_cnt;
};

// PT: pool element type, WT: wire element type, PACK: pool -> wire (else wire -> pool)
template <typename PT, typename WT, bool PACK>
__global__ __launch_bounds__(256) void wire_kernel(WireArgs a) {
    constexpr int kPer = kWirePer;
    const uint64_t g0 = (uint64_t)blockIdx.x * (256 * kPer) + threadIdx.x;
    using ST = typename std::conditional<PACK, PT, WT>::type; // what is read
    using DT = typename std::conditional<PACK, WT, PT>::type; // what is written
    Vec8<ST> in[kPer];
    uint64_t pool_off[kPer];
    const float* scale[kPer];
    bool live[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        const uint64_t g = g0 + (uint64_t)u * 256;
        live[u] = g < a.total_vecs;
        scale[u] = nullptr;
        if (!live[u]) continue;
        const uint32_t c = (uint32_t)(g / a.vecs_per_chunk), e = (uint32_t)(g % a.vecs_per_chunk) * 8;
        const uint32_t i = c / a.layer_cnt, l = c % a.layer_cnt;
        const int32_t page = a.page_ids[i];
        if ((uint64_t)(uint32_t)page >= a.max_pages) { // not a page of this pool: nothing is read from or written to
            live[u] = false;                           // the pool; a packed stream carries zeros in its place
            if (PACK) {
                Vec8<DT> z;
                z.raw = decltype(z.raw){};
                wire_store(z, reinterpret_cast<DT*>(a.wire) + g * 8);
            }
            continue;
        }
        pool_off[u] = ((uint64_t)(a.start_layer + l) * a.max_pages + (uint64_t)page) * a.stride_page + e;
        if (sizeof(PT) != sizeof(WT)) {
            const uint32_t half = (uint32_t)(a.stride_page / 2);
            const bool is_v = e >= half;
            const uint32_t head = (uint32_t)(((is_v ? e - half : e) / a.stride_h) % a.num_kv_heads);
            const float* sc = is_v ? a.v_scale : a.k_scale;
            if (sc) scale[u] = sc + (size_t)l * a.num_kv_heads + head;
        }
        const ST* src = PACK ? reinterpret_cast<const ST*>(a.pool) + pool_off[u]
                             : reinterpret_cast<const ST*>(a.wire) + g * 8;
        wire_load(in[u], src);
    }
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
        if (!live[u]) continue;
        const uint64_t g = g0 + (uint64_t)u * 256;
        DT* dst = PACK ? reinterpret_cast<DT*>(a.wire) + g * 8 : reinterpret_cast<DT*>(a.pool) + pool_off[u];
        if constexpr (sizeof(PT) == sizeof(WT)) {
            Vec8<DT> o;
            o.raw = in[u].raw; // bit copy
            wire_store(o, dst);
        } else {
            float x[8];
            in[u].to_float(x);
            if (scale[u]) {
                const float sc = *scale[u];
#pragma unroll
                for (int k = 0; k < 8; ++k) x[k] = PACK ? x[k] / sc : x[k] * sc;
            }
            Vec8<DT> o;
            o.from_float(x);
            wire_store(o, dst);
        }
    }
}

template <typename PT, typename WT, bool PACK>
static int launch_wire(const WireArgs& a, hipStream_t s) {
    const uint64_t per_wg = 256 * kWirePer;
    const uint64_t grid = (a.total_vecs + per_wg - 1) / per_wg;
    if (grid == 0) return 0;
    if (grid > 0x7fffffffull) return BZ_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((wire_kernel<PT, WT, PACK>), dim3((uint32_t)grid), dim3(256), 0, s, a);
    BZ_LAUNCH_CHECK();
    return 0;
}

template <bool PACK>
static int wire_dispatch(void* pool_base, uint64_t max_pages, const bz_paged_kv_t* kv, const int32_t* page_ids,
                         uint32_t num_pages, uint32_t start_layer, uint32_t layer_cnt, void* wire, int wire_dtype,
                         const float* k_scale, const float* v_scale, void* stream) {
    if (!kv) return BZ_ERR_BAD_ARG;
    if (num_pages == 0 || layer_cnt == 0) return 0;
    if (!pool_base || !page_ids || !wire) return BZ_ERR_BAD_ARG;
    if (kv->stride_page == 0 || kv->stride_page % 16 || kv->stride_h == 0 || kv->num_kv_heads == 0) return BZ_ERR_BAD_ARG;
    if (kv->stride_page / 8 > 0xffffffffull) return BZ_ERR_UNSUPPORTED;
    const int pd = kv->kv_dtype;
    if (pd != BZ_F16 && pd != BZ_BF16 && pd != BZ_E4M3) return BZ_ERR_BAD_ARG;
    if (wire_dtype != pd && !(wire_dtype == BZ_E4M3 && (pd == BZ_F16 || pd == BZ_BF16))) return BZ_ERR_UNSUPPORTED;
    WireArgs a;
    a.pool = (char*)pool_base;
    a.wire = (char*)wire;
    a.page_ids = page_ids;
    a.k_scale = k_scale;
    a.v_scale = v_scale;
    a.max_pages = max_pages;
    a.stride_page = kv->stride_page;
    a.stride_h = kv->stride_h;
    a.vecs_per_chunk = (uint32_t)(kv->stride_page / 8);
    a.total_vecs = (uint64_t)num_pages * layer_cnt * a.vecs_per_chunk;
    a.num_kv_heads = kv->num_kv_heads;
    a.start_layer = start_layer;
    a.layer_cnt = layer_cnt;
    hipStream_t s = (hipStream_t)stream;
    if (wire_dtype == pd) {
        // same element size on both sides: a bit copy whatever the type
        if (pd == BZ_E4M3) return launch_wire<e4m3_t, e4m3_t, PACK>(a, s);
        return launch_wire<f16_t, f16_t, PACK>(a, s);
    }
    if (pd == BZ_F16) return launch_wire<f16_t, e4m3_t, PACK>(a, s);
    return launch_wire<bf16_t, e4m3_t, PACK>(a, s);
}

} // namespace bz

using namespace bz;

extern "C" uint64_t bz_kv_wire_bytes(uint32_t num_pages, uint32_t layer_cnt, const bz_paged_kv_t* kv, int wire_dtype) {
    if (!kv) return 0;
    return (uint64_t)num_pages * layer_cnt * kv->stride_page * dtype_bytes(wire_dtype);
}

extern "C" int bz_kv_pages_pack(const void* pool_base, uint64_t max_pages, const bz_paged_kv_t* kv,
                                const int32_t* page_ids, uint32_t num_pages, uint32_t start_layer,
                                uint32_t layer_cnt, void* wire, int wire_dtype, const float* k_scale,
                                const float* v_scale, void* stream) {
    return wire_dispatch<true>(const_cast<void*>(pool_base), max_pages, kv, page_ids, num_pages, start_layer,
                               layer_cnt, wire, wire_dtype, k_scale, v_scale, stream);
}

extern "C" int bz_kv_pages_unpack(void* pool_base, uint64_t max_pages, const bz_paged_kv_t* kv,
                                  const int32_t* page_ids, uint32_t num_pages, uint32_t start_layer,
                                  uint32_t layer_cnt, const void* wire, int wire_dtype, const float* k_scale,
                                  const float* v_scale, void* stream) {
    return wire_dispatch<false>(pool_base, max_pages, kv, page_ids, num_pages, start_layer, layer_cnt,
                                const_cast<void*>(wire), wire_dtype, k_scale, v_scale, stream);
}
