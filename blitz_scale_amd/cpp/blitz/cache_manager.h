// KV pool owner, page allocator and host page-table maintenance: the integer semantics of
// src/blitz/cache_manager.h and of the page-table parts of src/blitz/batch.h of the BlitzScale
// worker, without their protobuf / tokenizer dependencies.
//
// Pool layout (one hipMalloc, sized for the 288 GB of an MI355X with 64-bit addressing):
//   [layer][page][K | V][head][slot][dim]   (BZ_LAYOUT_HND, default)   or
//   [layer][page][K | V][slot][head][dim]   (BZ_LAYOUT_NHD, the reference's order)
// A page's K and V of one layer stay one contiguous span of stride_page elements and layer planes
// are max_pages * stride_page apart, so the per-layer pointer bump of src/model/llama.h:378-381 and a
// per-(page, layer) transfer unit keep working.
#pragma once

#include <algorithm>
#include <cassert>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../kernel/page.h"

namespace blitz {

template<typename DType, typename IdType>
class CacheManager {
  public:
    static constexpr size_t kNumBatchMetaSlots = 256; // src/blitz/cache_manager.h:144-147

    /// with_device = false keeps everything on the host (no pool, malloc instead of pinned memory) so
    /// that the integer logic can run where there is no GPU.
    CacheManager(uint32_t local_num_kv_heads, uint32_t local_num_layers, uint32_t head_dim, uint32_t block_size,
                 uint32_t max_num_pages, int layout = BZ_LAYOUT_HND, bool with_device = true,
                 size_t meta_chunk_bytes = 2 * 1024 * 1024) :
        num_kv_heads_(local_num_kv_heads), num_layers_(local_num_layers), head_size_(head_dim), page_size_(block_size),
        max_num_page_(max_num_pages), layout_(layout), with_device_(with_device), chunk_bytes_(meta_chunk_bytes),
        free_mask_(max_num_pages, 1), meta_free_(kNumBatchMetaSlots, 1) {
        if (with_device_) {
            const uint64_t bytes = bz_kv_pool_bytes(num_layers_, max_num_page_, num_kv_heads_, page_size_, head_size_,
                                                    kernel::bz_dtype<DType>::value);
            kernel::bz_throw(bz_kv_pool_alloc(reinterpret_cast<void**>(&d_k_cache_), bytes), "KV pool alloc");
            if (hipHostMalloc(reinterpret_cast<void**>(&meta_), kNumBatchMetaSlots * chunk_bytes_, hipHostMallocDefault) !=
                hipSuccess)
                throw std::runtime_error("pinned page-table memory alloc failed");
        } else {
            meta_ = static_cast<IdType*>(std::malloc(kNumBatchMetaSlots * chunk_bytes_));
        }
    }
    CacheManager(const CacheManager&) = delete;
    CacheManager& operator=(const CacheManager&) = delete;
    ~CacheManager() {
        if (with_device_) {
            if (d_k_cache_) (void)bz_kv_pool_free(d_k_cache_);
            if (meta_) (void)hipHostFree(meta_);
        } else {
            std::free(meta_);
        }
    }

    /// src/blitz/cache_manager.h:197-253: take the lowest free page ids for every request, in request
    /// order, and write the blob [indices | indptr | last_page_len] into a free pinned chunk.
    void allocate(const std::vector<std::tuple<size_t, size_t>>& needed_blocks_slots, size_t num_blocks,
                  std::vector<IdType>& indices, std::vector<std::vector<IdType>>& indices_2d,
                  const std::vector<IdType>& indptr, const std::vector<IdType>& last_page_len, IdType** indices_h,
                  IdType** indptr_h, IdType** last_page_len_h, int* pinned_memory_idx) {
        assert(needed_blocks_slots.size() + 1 == indptr.size());
        assert(needed_blocks_slots.size() == last_page_len.size());
        const std::vector<IdType> fresh = first_fit(num_blocks); // throws before anything is marked
        // so does a table too large for its pinned chunk: checked here, before pages and the chunk are taken
        if ((indices.size() + num_blocks + indptr.size() + last_page_len.size()) * sizeof(IdType) > chunk_bytes_)
            throw std::runtime_error("page table does not fit its pinned chunk");
        const int meta = take_meta_slot();
        if (meta < 0) throw std::runtime_error("no free page-table chunk");
        *pinned_memory_idx = meta;
        size_t cursor = 0;
        for (const auto& [need_blocks, need_slots] : needed_blocks_slots) {
            (void)need_slots;
            std::vector<IdType> mine(fresh.begin() + cursor, fresh.begin() + cursor + need_blocks);
            for (IdType pg : mine) free_mask_[pg] = 0;
            indices.insert(indices.end(), mine.begin(), mine.end());
            indices_2d.emplace_back(std::move(mine));
            cursor += need_blocks;
            num_allocated_blocks_ += need_blocks;
        }
        flush(meta, indices, indptr, last_page_len, indices_h, indptr_h, last_page_len_h);
    }

    /// src/blitz/cache_manager.h:255-324: every sequence grows by one slot; a sequence whose last page
    /// is full gets the next lowest free page and starts it at slot 1.
    void append(std::vector<IdType>& indices, std::vector<std::vector<IdType>>& indices_2d, std::vector<IdType>& indptr,
                std::vector<IdType>& last_page_len, IdType** indices_h, IdType** indptr_h, IdType** last_page_len_h,
                const int pinned_memory_idx) {
        const size_t B = indices_2d.size();
        assert(last_page_len.size() == B);
        std::vector<size_t> full;
        for (size_t i = 0; i < B; ++i)
            if (last_page_len[i] == (IdType)page_size_) full.push_back(i);
        const std::vector<IdType> fresh = first_fit(full.size()); // all or nothing
        if ((indices.size() + full.size() + indptr.size() + last_page_len.size()) * sizeof(IdType) > chunk_bytes_)
            throw std::runtime_error("page table does not fit its pinned chunk");
        for (size_t i = 0; i < B; ++i)
            if (last_page_len[i] != (IdType)page_size_) last_page_len[i] += 1;
        if (full.empty()) {
            std::copy(last_page_len.begin(), last_page_len.end(), *last_page_len_h);
            return;
        }
        for (size_t i = 0; i < full.size(); ++i) {
            indices_2d[full[i]].push_back(fresh[i]);
            free_mask_[fresh[i]] = 0;
            last_page_len[full[i]] = 1;
        }
        num_allocated_blocks_ += full.size();
        indices.clear();
        indptr.assign(1, 0);
        for (size_t i = 0; i < B; ++i) {
            indices.insert(indices.end(), indices_2d[i].begin(), indices_2d[i].end());
            indptr.push_back((IdType)indices.size());
        }
        flush(pinned_memory_idx, indices, indptr, last_page_len, indices_h, indptr_h, last_page_len_h);
    }

    /// rewrite the pinned blob after the host vectors changed (filter / extend, src/blitz/batch.h:399-417,540-566)
    void flush(int meta, const std::vector<IdType>& indices, const std::vector<IdType>& indptr,
               const std::vector<IdType>& last_page_len, IdType** indices_h, IdType** indptr_h,
               IdType** last_page_len_h) {
        const size_t n = indices.size() + indptr.size() + last_page_len.size();
        if (n * sizeof(IdType) > chunk_bytes_) throw std::runtime_error("page table does not fit its pinned chunk");
        IdType* base = meta_ + (size_t)meta * (chunk_bytes_ / sizeof(IdType));
        std::copy(indices.begin(), indices.end(), base);
        std::copy(indptr.begin(), indptr.end(), base + indices.size());
        std::copy(last_page_len.begin(), last_page_len.end(), base + indices.size() + indptr.size());
        *indices_h = base;
        *indptr_h = base + indices.size();
        *last_page_len_h = base + indices.size() + indptr.size();
    }

    void free(const std::vector<IdType>& block_indices) {
        for (IdType pg : block_indices) free_mask_[pg] = 1;
        num_allocated_blocks_ -= block_indices.size();
    }
    void free_block_meta(int block_meta_idx) { meta_free_[block_meta_idx] = 1; }

    size_t get_free_block_num() const noexcept { return max_num_page_ - num_allocated_blocks_; }
    size_t get_allocated_block_num() const noexcept { return num_allocated_blocks_; }
    size_t get_total_block_num() const noexcept { return max_num_page_; }
    DType* get_base_ptr() const { return d_k_cache_; }
    std::tuple<void*, size_t> get_kvcache_segment() {
        return {d_k_cache_, (size_t)bz_kv_pool_bytes(num_layers_, max_num_page_, num_kv_heads_, page_size_, head_size_,
                                                     kernel::bz_dtype<DType>::value)};
    }
    kernel::PageTable<DType, IdType> empty_page_table(uint32_t batch_size) const noexcept {
        return kernel::PageTable<DType, IdType>{batch_size, page_size_, num_kv_heads_, head_size_, d_k_cache_, layout_};
    }
    /// base pointers of layer `layer` (the absolute form of the bump at src/model/llama.h:378-381)
    void set_layer(kernel::PageTable<DType, IdType>& pt, uint32_t layer) const {
        pt.k_data = d_k_cache_ + (size_t)layer * max_num_page_ * pt.stride_page;
        pt.v_data = pt.k_data + pt.stride_page / 2;
    }
    uint32_t page_size() const { return page_size_; }

  private:
    /// the lowest `n` free page ids (src/blitz/cache_manager.h:161-184); throws when fewer are free
    std::vector<IdType> first_fit(size_t n) const {
        std::vector<IdType> res;
        res.reserve(n);
        for (size_t i = 0; i < max_num_page_ && res.size() < n; ++i)
            if (free_mask_[i]) res.push_back((IdType)i);
        if (res.size() < n)
            throw std::runtime_error("Try to allocate " + std::to_string(n) + " blocks, but " +
                                     std::to_string(res.size()) + " is free!");
        return res;
    }
    int take_meta_slot() {
        for (size_t i = 0; i < kNumBatchMetaSlots; ++i)
            if (meta_free_[i]) { meta_free_[i] = 0; return (int)i; }
        return -1;
    }

    const uint32_t num_kv_heads_, num_layers_, head_size_, page_size_, max_num_page_;
    const int layout_;
    const bool with_device_;
    const size_t chunk_bytes_;
    size_t num_allocated_blocks_ = 0;
    std::vector<uint8_t> free_mask_, meta_free_;
    IdType* meta_ = nullptr;
    DType* d_k_cache_ = nullptr;
};

/// Host side of one batch's page table: what src/blitz/batch.h keeps next to the PageTable
/// (indices_2d, the pinned chunk id) and the operations that change it.
template<typename DType, typename IdType>
struct HostBatch {
    CacheManager<DType, IdType>* cm;
    kernel::PageTable<DType, IdType> page_table;
    std::vector<std::vector<IdType>> indices_2d;
    std::vector<IdType> ragged_indptr; // prompt offsets, prefill only
    int pinned_memory_idx = -1;

    /// prefill constructor rule (src/blitz/batch.h:236-257): a prompt of len tokens reserves len + 1 slots
    HostBatch(CacheManager<DType, IdType>* cm_, const std::vector<IdType>& prompt_lens) :
        cm(cm_), page_table(cm_->empty_page_table((uint32_t)prompt_lens.size())) {
        const size_t P = page_table.page_size;
        std::vector<std::tuple<size_t, size_t>> need;
        size_t blocks = 0;
        IdType tok = 0;
        for (IdType len : prompt_lens) {
            ragged_indptr.push_back(tok);
            tok += len;
            const size_t slots = (size_t)len + 1, nb = (slots + P - 1) / P;
            page_table.indptr.push_back((IdType)blocks);
            page_table.last_page_len.push_back((IdType)(slots - (nb - 1) * P));
            need.emplace_back(nb, slots);
            blocks += nb;
        }
        ragged_indptr.push_back(tok);
        page_table.indptr.push_back((IdType)blocks);
        cm->allocate(need, blocks, page_table.indices, indices_2d, page_table.indptr, page_table.last_page_len,
                     &page_table.indices_h, &page_table.indptr_h, &page_table.last_page_len_h, &pinned_memory_idx);
    }

    /// Batch::update's page-table half (src/blitz/batch.h:280-295)
    void grow() {
        cm->append(page_table.indices, indices_2d, page_table.indptr, page_table.last_page_len, &page_table.indices_h,
                   &page_table.indptr_h, &page_table.last_page_len_h, pinned_memory_idx);
    }

    /// Batch::filter's page-table half (src/blitz/batch.h:297-418): keep the listed sequences, in the
    /// listed (ascending) order, free the pages of the others
    void filter(const std::vector<size_t>& keep) {
        if (keep.empty()) throw std::runtime_error("Call filter batch with empty request_ids");
        std::vector<std::vector<IdType>> kept2d;
        std::vector<IdType> kept_lpl;
        std::vector<char> is_kept(indices_2d.size(), 0);
        for (size_t i : keep) is_kept[i] = 1;
        for (size_t i = 0; i < indices_2d.size(); ++i) {
            if (is_kept[i]) {
                kept2d.push_back(indices_2d[i]);
                kept_lpl.push_back(page_table.last_page_len[i]);
            } else {
                cm->free(indices_2d[i]);
            }
        }
        indices_2d = std::move(kept2d);
        page_table.last_page_len = std::move(kept_lpl);
        rebuild();
    }

    /// Batch::extend's page-table half (src/blitz/batch.h:482-576): concatenate other batches onto this one
    void extend(HostBatch& other) {
        indices_2d.insert(indices_2d.end(), other.indices_2d.begin(), other.indices_2d.end());
        page_table.last_page_len.insert(page_table.last_page_len.end(), other.page_table.last_page_len.begin(),
                                        other.page_table.last_page_len.end());
        cm->free_block_meta(other.pinned_memory_idx);
        other.indices_2d.clear();
        other.pinned_memory_idx = -1;
        rebuild();
    }

    /// release pages and the pinned chunk
    void release() {
        for (auto& pages : indices_2d) cm->free(pages);
        indices_2d.clear();
        if (pinned_memory_idx >= 0) cm->free_block_meta(pinned_memory_idx);
        pinned_memory_idx = -1;
    }

  private:
    void rebuild() {
        page_table.batch_size = (uint32_t)indices_2d.size();
        page_table.indices.clear();
        page_table.indptr.assign(1, 0);
        for (const auto& pages : indices_2d) {
            page_table.indices.insert(page_table.indices.end(), pages.begin(), pages.end());
            page_table.indptr.push_back((IdType)page_table.indices.size());
        }
        ragged_indptr.clear();
        cm->flush(pinned_memory_idx, page_table.indices, page_table.indptr, page_table.last_page_len,
                  &page_table.indices_h, &page_table.indptr_h, &page_table.last_page_len_h);
    }
};

} // namespace blitz
