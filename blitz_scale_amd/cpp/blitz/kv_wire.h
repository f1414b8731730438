// The data-format half of src/blitz/migration_manager.h of the BlitzScale worker: which bytes of the
// KV pool make up a batch's migration payload and in which order.  The transport (the reference's
// TcclSend / NCCL send per message) is not part of this library.
#pragma once

#include <cstddef>
#include <cstdint>

#include "../kernel/page.h"

namespace blitz {

template<typename DType, typename IdType>
class KvWire {
  public:
    /// kv_data: layer 0 of the pool (CacheManager::get_base_ptr()); max_num_pages: pages per layer plane
    KvWire(DType* kv_data, uint32_t max_num_pages) : kv_data_(kv_data), max_num_pages_(max_num_pages) {}

    /// src/blitz/migration_manager.h:86-92: the (page, layer) unit the reference sends as one message
    DType* get_page_ptr(const kernel::PageTable<DType, IdType>& page_table, size_t block_id, size_t curr_layer) const {
        DType* layer_base = kv_data_ + curr_layer * max_num_pages_ * page_table.stride_page;
        return layer_base + block_id * page_table.stride_page;
    }

    /// bytes of the payload of num_pages pages over layer_cnt layers
    size_t wire_bytes(const kernel::PageTable<DType, IdType>& page_table, uint32_t num_pages, uint32_t layer_cnt,
                      int wire_dtype = kernel::bz_dtype<DType>::value) const {
        const bz_paged_kv_t kv = page_table.c_view();
        return (size_t)bz_kv_wire_bytes(num_pages, layer_cnt, &kv, wire_dtype);
    }

    /// The messages of send_multi_layer_fast (src/blitz/migration_manager.h:455-467) for the pages
    /// page_ids_d[0..num_pages) (device array: a batch's prompt blocks, request by request) and layers
    /// start_layer .. start_layer + layer_cnt - 1, concatenated into `wire`: message (i, l) starts at
    /// element (i*layer_cnt + l) * stride_page.  With wire_dtype BZ_E4M3 on a 16-bit pool the elements
    /// travel as e4m3(x / scale), scales [layer_cnt][num_heads] per K and V (device, may be null).
    void pack(const kernel::PageTable<DType, IdType>& page_table, const IdType* page_ids_d, uint32_t num_pages,
              uint32_t start_layer, uint32_t layer_cnt, void* wire, int wire_dtype = kernel::bz_dtype<DType>::value,
              const float* k_scale = nullptr, const float* v_scale = nullptr) const {
        static_assert(sizeof(IdType) == 4, "page ids are int32");
        const bz_paged_kv_t kv = page_table.c_view();
        kernel::bz_throw(bz_kv_pages_pack(kv_data_, max_num_pages_, &kv, reinterpret_cast<const int32_t*>(page_ids_d),
                                          num_pages, start_layer, layer_cnt, wire, wire_dtype, k_scale, v_scale,
                                          page_table.opts().stream),
                         "PackKVPages");
    }

    /// The receiving side (recv loops of src/blitz/migration_manager.h mirror the send order): message
    /// (i, l) of `wire` goes to page page_ids_d[i] of layer start_layer + l of this pool.
    void unpack(const kernel::PageTable<DType, IdType>& page_table, const IdType* page_ids_d, uint32_t num_pages,
                uint32_t start_layer, uint32_t layer_cnt, const void* wire,
                int wire_dtype = kernel::bz_dtype<DType>::value, const float* k_scale = nullptr,
                const float* v_scale = nullptr) const {
        static_assert(sizeof(IdType) == 4, "page ids are int32");
        const bz_paged_kv_t kv = page_table.c_view();
        kernel::bz_throw(bz_kv_pages_unpack(kv_data_, max_num_pages_, &kv,
                                            reinterpret_cast<const int32_t*>(page_ids_d), num_pages, start_layer,
                                            layer_cnt, wire, wire_dtype, k_scale, v_scale,
                                            page_table.opts().stream),
                         "UnpackKVPages");
    }

  private:
    DType* kv_data_;
    uint32_t max_num_pages_;
};

} // namespace blitz
