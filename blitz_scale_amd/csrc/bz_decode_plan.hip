// Host-side decode planner: replaces BlitzBatchDecodeHandler::plan
// (src/kernel/flashinfer_types.cu:52-80 of the BlitzScale worker).  Pure integer work on the
// host copies of the page table plus one asynchronous upload of the schedule.
#include <algorithm>
#include <cstring>
#include <new>
#include <vector>

#include "bz_common.hpp"
#include "bz_decode_plan.hpp"

namespace bz {

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

static int device_cu_count() {
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
    }
    return cus;
}

} // namespace bz

using namespace bz;

extern "C" bz_decode_plan_t* bz_decode_plan_create(void) {
    DecodePlan* p = new (std::nothrow) DecodePlan();
    return reinterpret_cast<bz_decode_plan_t*>(p);
}

extern "C" void bz_decode_plan_destroy(bz_decode_plan_t* plan_) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p) return;
    if (p->upload_done) {
        (void)hipEventSynchronize(p->upload_done);
        (void)hipEventDestroy(p->upload_done);
    }
    if (p->staging) (void)hipHostFree(p->staging);
    delete p;
}

extern "C" int bz_decode_plan(bz_decode_plan_t* plan_, void* float_buffer, size_t float_buffer_bytes,
                              void* int_buffer, size_t int_buffer_bytes, const int32_t* indptr_h,
                              const int32_t* last_page_len_h, uint32_t batch_size, uint32_t num_qo_heads,
                              uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size, uint32_t split_tokens,
                              void* stream) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p || !indptr_h || !last_page_len_h || !float_buffer || !int_buffer) return BZ_ERR_BAD_ARG;
    if (page_size == 0 || num_kv_heads == 0 || num_qo_heads % num_kv_heads) return BZ_ERR_BAD_ARG;
    p->planned = false;
    if (split_tokens == 0) split_tokens = 2048;

    // ---- choose the piece length (in pages) -------------------------------------------------
    // Pieces never exceed split_tokens (contexts longer than that are always split); they are
    // shortened further, down to 256 tokens, until the launch holds about four workgroups per CU.
    const int cus = device_cu_count();
    const uint32_t max_pages_cap = std::max<uint32_t>(1, split_tokens / page_size);
    const uint32_t min_pages = std::min<uint32_t>(max_pages_cap, std::max<uint32_t>(1, 256 / page_size));
    uint32_t piece = max_pages_cap;
    auto count_items = [&](uint32_t pc) {
        uint64_t n = 0;
        for (uint32_t b = 0; b < batch_size; ++b) {
            const int32_t np = indptr_h[b + 1] - indptr_h[b];
            if (np > 0) n += ((uint32_t)np + pc - 1) / pc;
        }
        return n * num_kv_heads;
    };
    // split_tokens == UINT32_MAX switches splitting off altogether (one piece per sequence)
    const bool never_split = split_tokens == 0xffffffffu;
    while (!never_split && piece > min_pages && count_items(piece) < (uint64_t)cus * 4)
        piece = std::max(min_pages, piece / 2);

    std::vector<DecodeSegment> segs;
    std::vector<DecodeCombine> combos;
    std::vector<int32_t> empty;
    uint32_t partials = 0;
    for (uint32_t b = 0; b < batch_size; ++b) {
        const int32_t np = indptr_h[b + 1] - indptr_h[b];
        if (np < 0) return BZ_ERR_BAD_ARG;
        if (np == 0) { empty.push_back((int32_t)b); continue; }
        if (last_page_len_h[b] < 1 || last_page_len_h[b] > (int32_t)page_size) return BZ_ERR_BAD_ARG;
        const uint32_t n = ((uint32_t)np + piece - 1) / piece;
        if (n == 1) {
            segs.push_back({(int32_t)b, 0, np, -1});
        } else {
            // equal pieces rather than (piece, piece, ..., remainder): same count, better balance
            combos.push_back({(int32_t)b, (int32_t)partials, (int32_t)n, 0});
            for (uint32_t i = 0; i < n; ++i) {
                const int32_t lo = (int32_t)((uint64_t)np * i / n), hi = (int32_t)((uint64_t)np * (i + 1) / n);
                segs.push_back({(int32_t)b, lo, hi, (int32_t)(partials + i)});
            }
            partials += n;
        }
    }
    // longest pieces first: the dispatcher hands workgroups out in order, so the tail is short
    std::stable_sort(segs.begin(), segs.end(), [](const DecodeSegment& x, const DecodeSegment& y) {
        return (x.page_end - x.page_begin) > (y.page_end - y.page_begin);
    });

    // ---- workspaces -------------------------------------------------------------------------
    const size_t seg_bytes = align_up(segs.size() * sizeof(DecodeSegment), 256);
    const size_t combo_bytes = align_up(combos.size() * sizeof(DecodeCombine), 256);
    const size_t empty_bytes = align_up(empty.size() * sizeof(int32_t), 256);
    const size_t total = seg_bytes + combo_bytes + empty_bytes;
    if (total > int_buffer_bytes) return BZ_ERR_WORKSPACE;
    const size_t part_o_bytes = align_up((size_t)partials * num_qo_heads * head_dim * sizeof(float), 256);
    const size_t part_lse_bytes = align_up((size_t)partials * num_qo_heads * sizeof(float), 256);
    if (part_o_bytes + part_lse_bytes > float_buffer_bytes) return BZ_ERR_WORKSPACE;

    hipStream_t s = (hipStream_t)stream;
    if (!p->upload_done) BZ_CHECK_HIP(hipEventCreateWithFlags(&p->upload_done, hipEventDisableTiming));
    else BZ_CHECK_HIP(hipEventSynchronize(p->upload_done)); // previous upload may still read staging
    if (total > p->staging_bytes) {
        if (p->staging) BZ_CHECK_HIP(hipHostFree(p->staging));
        p->staging = nullptr;
        p->staging_bytes = 0;
        const size_t want = std::max<size_t>(align_up(total * 2, 4096), 1 << 16);
        BZ_CHECK_HIP(hipHostMalloc(&p->staging, want, hipHostMallocDefault));
        p->staging_bytes = want;
    }
    char* st = (char*)p->staging;
    if (total) memset(st, 0, total);
    if (!segs.empty()) memcpy(st, segs.data(), segs.size() * sizeof(DecodeSegment));
    if (!combos.empty()) memcpy(st + seg_bytes, combos.data(), combos.size() * sizeof(DecodeCombine));
    if (!empty.empty()) memcpy(st + seg_bytes + combo_bytes, empty.data(), empty.size() * sizeof(int32_t));
    if (total) BZ_CHECK_HIP(hipMemcpyAsync(int_buffer, st, total, hipMemcpyHostToDevice, s));
    BZ_CHECK_HIP(hipEventRecord(p->upload_done, s));

    p->segments_d = (const DecodeSegment*)int_buffer;
    p->combos_d = (const DecodeCombine*)((char*)int_buffer + seg_bytes);
    p->empty_d = (const int32_t*)((char*)int_buffer + seg_bytes + combo_bytes);
    p->part_o = (float*)float_buffer;
    p->part_lse = (float*)((char*)float_buffer + part_o_bytes);
    p->batch_size = batch_size; p->num_qo_heads = num_qo_heads; p->num_kv_heads = num_kv_heads;
    p->head_dim = head_dim; p->page_size = page_size;
    p->num_segments = (uint32_t)segs.size(); p->num_combos = (uint32_t)combos.size();
    p->num_empty = (uint32_t)empty.size(); p->num_partials = partials;
    p->num_workgroups = (uint32_t)segs.size() * num_kv_heads;
    p->planned = true;
    return 0;
}

extern "C" int bz_decode_plan_info(const bz_decode_plan_t* plan_, uint32_t* num_segments, uint32_t* num_split_seqs,
                                   uint32_t* num_workgroups) {
    const DecodePlan* p = reinterpret_cast<const DecodePlan*>(plan_);
    if (!p || !p->planned) return BZ_ERR_NOT_PLANNED;
    if (num_segments) *num_segments = p->num_segments;
    if (num_split_seqs) *num_split_seqs = p->num_combos;
    if (num_workgroups) *num_workgroups = p->num_workgroups;
    return 0;
}
