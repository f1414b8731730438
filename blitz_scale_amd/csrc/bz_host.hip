// C ABI over the host-side page-table logic (blitz_scale_amd/cpp/blitz/cache_manager.h): pool
// ownership, first-fit page allocation, the prefill len+1 reservation, per-step growth, filter and
// extend.  Pure host code; replaces the page-table parts of src/blitz/cache_manager.h and
// src/blitz/batch.h of the BlitzScale worker.
#include <memory>
#include <new>
#include <vector>

#include "../cpp/blitz/cache_manager.h"

namespace {

struct CmBase {
    virtual ~CmBase() = default;
    virtual int prefill(const int32_t* lens, uint32_t n) = 0;
    virtual void grow(int id) = 0;
    virtual void filter(int id, const uint32_t* keep, uint32_t n) = 0;
    virtual void extend(int dst, int src) = 0;
    virtual void release(int id) = 0;
    virtual void table(int id, const int32_t** ind, uint32_t* nnz, const int32_t** ip, const int32_t** lpl,
                       uint32_t* batch) = 0;
    virtual void stats(uint64_t* free_p, uint64_t* alloc_p, uint64_t* total_p) = 0;
    virtual void pool(void** base, uint64_t* bytes) = 0;
};

template<typename DType>
struct CmImpl : CmBase {
    blitz::CacheManager<DType, int32_t> cm;
    std::vector<std::unique_ptr<blitz::HostBatch<DType, int32_t>>> batches;

    CmImpl(uint32_t h, uint32_t l, uint32_t d, uint32_t p, uint32_t pages, int layout, bool dev, size_t chunk) :
        cm(h, l, d, p, pages, layout, dev, chunk) {}

    blitz::HostBatch<DType, int32_t>& at(int id) {
        if (id < 0 || (size_t)id >= batches.size() || !batches[id]) throw std::out_of_range("unknown batch id");
        return *batches[id];
    }
    int prefill(const int32_t* lens, uint32_t n) override {
        std::vector<int32_t> v(lens, lens + n);
        auto b = std::make_unique<blitz::HostBatch<DType, int32_t>>(&cm, v);
        for (size_t i = 0; i < batches.size(); ++i)
            if (!batches[i]) { batches[i] = std::move(b); return (int)i; }
        batches.push_back(std::move(b));
        return (int)batches.size() - 1;
    }
    void grow(int id) override { at(id).grow(); }
    void filter(int id, const uint32_t* keep, uint32_t n) override {
        std::vector<size_t> k(keep, keep + n);
        for (size_t i : k)
            if (i >= at(id).indices_2d.size()) throw std::out_of_range("filter index");
        at(id).filter(k);
    }
    void extend(int dst, int src) override {
        if (dst == src) throw std::invalid_argument("extend onto itself");
        at(dst).extend(at(src));
        batches[src].reset();
    }
    void release(int id) override {
        at(id).release();
        batches[id].reset();
    }
    void table(int id, const int32_t** ind, uint32_t* nnz, const int32_t** ip, const int32_t** lpl,
               uint32_t* batch) override {
        auto& b = at(id);
        if (ind) *ind = b.page_table.indices_h;
        if (nnz) *nnz = (uint32_t)b.page_table.indices.size();
        if (ip) *ip = b.page_table.indptr_h;
        if (lpl) *lpl = b.page_table.last_page_len_h;
        if (batch) *batch = b.page_table.batch_size;
    }
    void stats(uint64_t* free_p, uint64_t* alloc_p, uint64_t* total_p) override {
        if (free_p) *free_p = cm.get_free_block_num();
        if (alloc_p) *alloc_p = cm.get_allocated_block_num();
        if (total_p) *total_p = cm.get_total_block_num();
    }
    void pool(void** base, uint64_t* bytes) override {
        auto [p, n] = cm.get_kvcache_segment();
        if (base) *base = p;
        if (bytes) *bytes = n;
    }
};

template<typename F>
int guarded(F&& f) {
    try {
        f();
        return 0;
    } catch (const std::out_of_range&) {
        return BZ_ERR_BAD_ARG;
    } catch (const std::invalid_argument&) {
        return BZ_ERR_BAD_ARG;
    } catch (const std::bad_alloc&) {
        return (int)hipErrorOutOfMemory;
    } catch (const std::runtime_error&) {
        return BZ_ERR_NO_PAGES; // allocator exhaustion (src/blitz/cache_manager.h:174-182) or a full chunk
    }
}

} // namespace

extern "C" int bz_cm_create(bz_cache_manager_t** out, uint32_t num_kv_heads, uint32_t num_layers, uint32_t head_dim,
                            uint32_t page_size, uint32_t max_pages, int kv_dtype, int layout, int with_device) {
    if (!out || !num_kv_heads || !num_layers || !head_dim || !page_size || !max_pages) return BZ_ERR_BAD_ARG;
    const size_t chunk = with_device ? (size_t)2 << 20 : (size_t)256 << 10;
    return guarded([&] {
        CmBase* p = nullptr;
        if (kv_dtype == BZ_F16)
            p = new CmImpl<__half>(num_kv_heads, num_layers, head_dim, page_size, max_pages, layout, with_device != 0, chunk);
        else if (kv_dtype == BZ_BF16)
            p = new CmImpl<__hip_bfloat16>(num_kv_heads, num_layers, head_dim, page_size, max_pages, layout,
                                           with_device != 0, chunk);
        else if (kv_dtype == BZ_E4M3)
            p = new CmImpl<blitz::kernel::e4m3_storage>(num_kv_heads, num_layers, head_dim, page_size, max_pages, layout,
                                                        with_device != 0, chunk);
        else
            throw std::invalid_argument("kv dtype");
        *out = reinterpret_cast<bz_cache_manager_t*>(p);
    });
}

extern "C" void bz_cm_destroy(bz_cache_manager_t* cm) { delete reinterpret_cast<CmBase*>(cm); }

#define BZ_CM(cm) (*reinterpret_cast<CmBase*>(cm))

extern "C" int bz_cm_batch_prefill(bz_cache_manager_t* cm, const int32_t* prompt_lens, uint32_t batch, int* batch_id) {
    if (!cm || !prompt_lens || !batch_id) return BZ_ERR_BAD_ARG;
    return guarded([&] { *batch_id = BZ_CM(cm).prefill(prompt_lens, batch); });
}
extern "C" int bz_cm_batch_grow(bz_cache_manager_t* cm, int batch_id) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).grow(batch_id); });
}
extern "C" int bz_cm_batch_filter(bz_cache_manager_t* cm, int batch_id, const uint32_t* keep, uint32_t n_keep) {
    if (!cm || !keep) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).filter(batch_id, keep, n_keep); });
}
extern "C" int bz_cm_batch_extend(bz_cache_manager_t* cm, int dst_batch_id, int src_batch_id) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).extend(dst_batch_id, src_batch_id); });
}
extern "C" int bz_cm_batch_release(bz_cache_manager_t* cm, int batch_id) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).release(batch_id); });
}
extern "C" int bz_cm_batch_table(bz_cache_manager_t* cm, int batch_id, const int32_t** indices_h, uint32_t* nnz_pages,
                                 const int32_t** indptr_h, const int32_t** last_page_len_h, uint32_t* batch) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).table(batch_id, indices_h, nnz_pages, indptr_h, last_page_len_h, batch); });
}
extern "C" int bz_cm_stats(bz_cache_manager_t* cm, uint64_t* free_pages, uint64_t* allocated_pages,
                           uint64_t* total_pages) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).stats(free_pages, allocated_pages, total_pages); });
}
extern "C" int bz_cm_pool(bz_cache_manager_t* cm, void** base, uint64_t* bytes) {
    if (!cm) return BZ_ERR_BAD_ARG;
    return guarded([&] { BZ_CM(cm).pool(base, bytes); });
}
