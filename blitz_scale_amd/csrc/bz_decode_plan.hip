// Host-side decode planner: replaces BlitzBatchDecodeHandler::plan
// (src/kernel/flashinfer_types.cu:52-80 of the BlitzScale worker).  Pure integer work on the
// host copies of the page table plus one asynchronous upload of the schedule.
#include <algorithm>
#include <cstdlib>
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

namespace bz {

struct ScheduleCounts {
    uint32_t partials = 0, mfma_partials = 0;
    bool mfma_shape = false;
};

// Section sizes of the schedule inside the two workspaces (each section 256-byte aligned).
struct ScheduleLayout {
    size_t seg_bytes, combo_bytes, empty_bytes, base_total, part_o_bytes, part_lse_bytes;
    size_t mp_bytes, nheads, mptr_bytes, mc_bytes, cnt_bytes, mpart_o_bytes, mpart_lse_bytes;
    size_t unit_bytes, step_part_o_bytes, step_part_lse_bytes; // one-call decode step: unit list, one partial per piece
};

// Pure host work: fills the plan's host scratch (h_*) from the host copies of the page table.
static int build_schedule(DecodePlan* p, const int32_t* indptr_h, const int32_t* last_page_len_h, uint32_t batch_size,
                          uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size,
                          uint32_t split_tokens, int cus, ScheduleCounts* counts) {
    if (split_tokens == 0) split_tokens = 2048;
    // ---- choose the piece length (in pages) -------------------------------------------------
    // Pieces never exceed split_tokens (contexts longer than that are always split); they are
    // shortened further, down to 256 tokens, until the launch holds about four workgroups per CU.
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

    std::vector<DecodeSegment>& segs = p->h_segs;
    std::vector<DecodeCombine>& combos = p->h_combos;
    std::vector<int32_t>& empty = p->h_empty;
    segs.clear(); combos.clear(); empty.clear();
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

    // ---- MFMA path schedule ---------------------------------------------------------------------
    // The flattened (sequence, kv head, 32-token tile) space is divided into equal shares, one per
    // wave slot of the chip (8 single-wave workgroups per CU).  A share that crosses a (sequence, kv
    // head) boundary becomes several pieces; a (sequence, kv head) that ends up in more than one
    // piece, or is longer than split_tokens, is folded from partial results.  Every tile of a share
    // gets a 16-byte record so that the kernel never has to chase the piece list tile by tile.
    std::vector<MfmaPiece>& mp = p->h_pieces;
    RawArray<MfmaTile>& mt = p->h_tiles;
    std::vector<int32_t>& mptr = p->h_slot_ptr; // tiles of slot s: [mptr[s], mptr[s+1]); uploaded as one MfmaSlotHead per slot
    std::vector<MfmaCombine>& mc = p->h_mcombos;
    std::vector<MfmaUnit>& mu = p->h_units;
    mp.clear(); mt.clear(); mptr.clear(); mc.clear(); mu.clear();
    uint32_t mfma_partials = 0;
    // A group of more than 16 q heads per kv head does not fit the 16 columns of the score tile: it is
    // scheduled as `parts` equal parts, each a kv head of its own as far as the schedule goes (heads
    // [u*gp, (u+1)*gp) of unit u = kvh*parts + part; the K/V of the kv head are read once per part).
    const uint32_t group = num_qo_heads / num_kv_heads;
    uint32_t parts = (group + 15) / 16;
    while (parts < group && group % parts) ++parts;
    const bool mfma_shape = head_dim == 128 && page_size % 16 == 0 && group / parts <= 16 && parts <= 8;
    p->mfma_parts = mfma_shape ? parts : 1;
    const uint32_t num_units = num_kv_heads * (mfma_shape ? parts : 1); // kv heads as the matrix-core schedule sees them
    if (mfma_shape) {
        uint64_t total_tiles = 0;
        for (uint32_t b = 0; b < batch_size; ++b) {
            const int32_t np = indptr_h[b + 1] - indptr_h[b];
            if (np <= 0) continue;
            const int64_t len = (int64_t)(np - 1) * page_size + last_page_len_h[b];
            total_tiles += (uint64_t)((len + 31) / 32) * num_units;
        }
        int page_shift = -1; // log2(page_size) when it is a power of two
        if ((page_size & (page_size - 1)) == 0) { page_shift = 0; while ((1u << page_shift) < page_size) ++page_shift; }
        const uint64_t max_slots = (uint64_t)cus * 8;
        const uint64_t share = std::max<uint64_t>(1, (total_tiles + max_slots - 1) / max_slots);
        p->mfma_streaming = share >= 2;
        const uint32_t cap_tiles = never_split ? 0x7fffffffu : std::max<uint32_t>(1, split_tokens / 32);
        // Workgroups are dealt round-robin to the 8 XCDs.  With plain K/V loads the odd XCDs streamed HBM
        // about a tenth slower than the even ones under full load (measured per wave with wall_clock64)
        // and a 9 % smaller share for their slots paid; with the non-temporal loads of the streaming
        // kernel the difference is gone and equal shares are fastest (128 x 32/8 heads bf16: 107.8 us at
        // 0 %, 108.7 at 3 %, 110.2 at 9 %, 108.3 at -4 %).  BZ_DECODE_XCD_SKEW sets the percentage.
        double skew = 0.0;
        if (const char* e = getenv("BZ_DECODE_XCD_SKEW")) skew = atof(e) / 100.0;
        if (share < 8) skew = 0.0; // too few tiles per slot to express the difference
        const uint64_t nslots = std::min<uint64_t>(max_slots, (total_tiles + share - 1) / share);
        auto slot_weight = [&](uint64_t s) { return (s & 1) ? 1.0 - skew / 2 : 1.0 + skew / 2; };
        double wsum = 0.0;
        for (uint64_t s2 = 0; s2 < nslots; ++s2) wsum += slot_weight(s2);
        const double tiles_per_weight = wsum > 0.0 ? (double)total_tiles / wsum : 0.0;
        uint64_t slot = 0, bound_lo = 0; // bound_lo: rounded running boundary where the current slot starts
        double wacc = slot_weight(0);
        auto slot_share = [&](void) { // tiles of the current slot: difference of rounded running boundaries
            const uint64_t hi = (slot + 1 >= nslots) ? total_tiles : (uint64_t)(wacc * tiles_per_weight + 0.5);
            const uint64_t lo = bound_lo;
            bound_lo = hi;
            return std::max<uint64_t>(1, hi > lo ? hi - lo : 1);
        };
        uint64_t room = slot_share(); // tiles the current slot can still take
        mt.resize_uninitialized(total_tiles); // sized once; every record is written below
        size_t n_rec = 0;
        mptr.push_back(0);
        for (uint32_t b = 0; b < batch_size; ++b) {
            const int32_t np = indptr_h[b + 1] - indptr_h[b];
            if (np <= 0) continue;
            const int64_t len = (int64_t)(np - 1) * page_size + last_page_len_h[b];
            const int32_t tiles = (int32_t)((len + 31) / 32);
            for (uint32_t h = 0; h < num_units; ++h) {
                const size_t first_piece = mp.size();
                int32_t t = 0;
                while (t < tiles) {
                    if (room == 0) {
                        mptr.push_back((int32_t)n_rec);
                        ++slot;
                        wacc += slot_weight(slot);
                        room = slot_share();
                    }
                    const uint64_t left = (uint64_t)(tiles - t);
                    const int32_t take = never_split ? (int32_t)left
                                                     : (int32_t)std::min<uint64_t>({left, room, (uint64_t)cap_tiles});
                    room -= std::min<uint64_t>(room, (uint64_t)take);
                    // one record per tile; page sizes are powers of two in practice, so the two page
                    // indices of a tile come from shifts rather than 64-bit divisions
                    MfmaTile* rec = mt.data() + n_rec;
                    n_rec += (size_t)take;
                    const int32_t piece_id = (int32_t)mp.size(), ip0 = indptr_h[b];
                    if (page_shift >= 0) {
                        // tiles whose second half still lies inside the table need no clamping: plain
                        // 32-bit shifts the compiler can vectorise; the (at most one) tile after them is clamped
                        const int64_t cap_tok = ((int64_t)np << page_shift) - 17;
                        const int32_t fast_end = cap_tok < 0 ? t : (int32_t)std::min<int64_t>(t + take, cap_tok / 32 + 1);
                        int32_t tt = t;
                        if ((int64_t)(t + take) * 32 + 16 < 0x7fffffffLL) {
                            for (; tt < fast_end; ++tt, ++rec)
                                *rec = {ip0 + ((tt << 5) >> page_shift), ip0 + (((tt << 5) + 16) >> page_shift), tt, piece_id};
                        }
                        for (; tt < t + take; ++tt, ++rec) {
                            const int32_t pg0 = std::min<int32_t>((int32_t)(((int64_t)tt * 32) >> page_shift), np - 1);
                            const int32_t pg1 = std::min<int32_t>((int32_t)(((int64_t)tt * 32 + 16) >> page_shift), np - 1);
                            *rec = {ip0 + pg0, ip0 + pg1, tt, piece_id};
                        }
                    } else {
                        for (int32_t tt = t; tt < t + take; ++tt, ++rec) {
                            const int32_t pg0 = std::min<int32_t>((int32_t)(((int64_t)tt * 32) / page_size), np - 1);
                            const int32_t pg1 = std::min<int32_t>((int32_t)(((int64_t)tt * 32 + 16) / page_size), np - 1);
                            *rec = {ip0 + pg0, ip0 + pg1, tt, piece_id};
                        }
                    }
                    mp.push_back({(int32_t)b, (int32_t)h, t, t + take, -1, -1, 0, 0, indptr_h[b], np, (int32_t)len,
                                  (int32_t)(h / p->mfma_parts), {0, 0, 0, 0}});
                    t += take;
                }
                const size_t cnt = mp.size() - first_piece;
                mu.push_back({(int32_t)b, (int32_t)h, (int32_t)first_piece, (int32_t)cnt, indptr_h[b], (int32_t)len, {0, 0}});
                if (cnt > 1) {
                    mc.push_back({(int32_t)b, (int32_t)h, (int32_t)mfma_partials, (int32_t)cnt});
                    for (size_t i = 0; i < cnt; ++i) {
                        MfmaPiece& pc = mp[first_piece + i];
                        pc.partial = (int32_t)(mfma_partials + i);
                        pc.combo = (int32_t)mc.size() - 1;
                        pc.count = (int32_t)cnt;
                        pc.first = (int32_t)mfma_partials;
                    }
                    mfma_partials += (uint32_t)cnt;
                }
            }
        }
        mptr.push_back((int32_t)n_rec);
    }

    counts->partials = partials;
    counts->mfma_partials = mfma_partials;
    counts->mfma_shape = mfma_shape;
    return 0;
}

static ScheduleLayout schedule_layout(const DecodePlan* p, const ScheduleCounts& c, uint32_t num_qo_heads,
                                      uint32_t head_dim) {
    ScheduleLayout L;
    L.seg_bytes = align_up(p->h_segs.size() * sizeof(DecodeSegment), 256);
    L.combo_bytes = align_up(p->h_combos.size() * sizeof(DecodeCombine), 256);
    L.empty_bytes = align_up(p->h_empty.size() * sizeof(int32_t), 256);
    L.base_total = L.seg_bytes + L.combo_bytes + L.empty_bytes;
    L.part_o_bytes = align_up((size_t)c.partials * num_qo_heads * head_dim * sizeof(float), 256);
    L.part_lse_bytes = align_up((size_t)c.partials * num_qo_heads * sizeof(float), 256);
    L.mp_bytes = align_up(p->h_pieces.size() * sizeof(MfmaPiece), 256);
    L.nheads = p->h_slot_ptr.empty() ? 0 : p->h_slot_ptr.size() - 1;
    L.mptr_bytes = align_up(L.nheads * sizeof(MfmaSlotHead), 256); // slot heads
    L.mc_bytes = align_up(p->h_mcombos.size() * sizeof(MfmaCombine), 256);
    L.cnt_bytes = align_up(p->h_tiles.size() * sizeof(MfmaTile), 256); // tile records
    L.mpart_o_bytes = align_up((size_t)c.mfma_partials * 16 * 128 * sizeof(float), 256);
    L.mpart_lse_bytes = align_up((size_t)c.mfma_partials * 16 * sizeof(float), 256);
    L.unit_bytes = align_up(p->h_units.size() * sizeof(MfmaUnit), 256);
    L.step_part_o_bytes = align_up(p->h_pieces.size() * 16 * 128 * sizeof(float), 256);
    L.step_part_lse_bytes = align_up(p->h_pieces.size() * 16 * sizeof(float), 256);
    return L;
}

} // namespace bz

extern "C" int bz_decode_plan(bz_decode_plan_t* plan_, void* float_buffer, size_t float_buffer_bytes,
                              void* int_buffer, size_t int_buffer_bytes, const int32_t* indptr_h,
                              const int32_t* last_page_len_h, uint32_t batch_size, uint32_t num_qo_heads,
                              uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size, uint32_t split_tokens,
                              void* stream) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p || !indptr_h || !last_page_len_h || !float_buffer || !int_buffer) return BZ_ERR_BAD_ARG;
    if (page_size == 0 || num_kv_heads == 0 || num_qo_heads % num_kv_heads) return BZ_ERR_BAD_ARG;
    p->planned = false;
    ScheduleCounts counts;
    const int rc = build_schedule(p, indptr_h, last_page_len_h, batch_size, num_qo_heads, num_kv_heads, head_dim,
                                  page_size, split_tokens, device_cu_count(), &counts);
    if (rc) return rc;
    const std::vector<DecodeSegment>& segs = p->h_segs;
    const std::vector<DecodeCombine>& combos = p->h_combos;
    const std::vector<int32_t>& empty = p->h_empty;
    const std::vector<MfmaPiece>& mp = p->h_pieces;
    const RawArray<MfmaTile>& mt = p->h_tiles;
    const std::vector<int32_t>& mptr = p->h_slot_ptr;
    const std::vector<MfmaCombine>& mc = p->h_mcombos;
    const uint32_t partials = counts.partials, mfma_partials = counts.mfma_partials;
    const bool mfma_shape = counts.mfma_shape;

    // ---- workspaces -------------------------------------------------------------------------
    const ScheduleLayout L = schedule_layout(p, counts, num_qo_heads, head_dim);
    const size_t seg_bytes = L.seg_bytes, combo_bytes = L.combo_bytes, base_total = L.base_total;
    const size_t part_o_bytes = L.part_o_bytes, part_lse_bytes = L.part_lse_bytes;
    const size_t mp_bytes = L.mp_bytes, nheads = L.nheads, mptr_bytes = L.mptr_bytes, mc_bytes = L.mc_bytes;
    const size_t cnt_bytes = L.cnt_bytes, mpart_o_bytes = L.mpart_o_bytes, mpart_lse_bytes = L.mpart_lse_bytes;
    if (base_total > int_buffer_bytes) return BZ_ERR_WORKSPACE;
    if (part_o_bytes + part_lse_bytes > float_buffer_bytes) return BZ_ERR_WORKSPACE;
    // the MFMA schedule is optional: without room for it the general kernel runs
    const bool mfma_ok = mfma_shape && !mp.empty() && base_total + mp_bytes + mptr_bytes + mc_bytes + cnt_bytes <= int_buffer_bytes &&
                         mpart_o_bytes + mpart_lse_bytes <= float_buffer_bytes;
    const size_t mfma_total = base_total + mp_bytes + mptr_bytes + mc_bytes + cnt_bytes;
    // the unit list of the one-call decode step is optional on top of that
    const bool units_ok = mfma_ok && mfma_total + L.unit_bytes <= int_buffer_bytes;
    const size_t total = mfma_ok ? mfma_total + (units_ok ? L.unit_bytes : 0) : base_total;

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
    // (the padding between the 256-byte aligned sections is never read: no need to clear the buffer)
    if (!segs.empty()) memcpy(st, segs.data(), segs.size() * sizeof(DecodeSegment));
    if (!combos.empty()) memcpy(st + seg_bytes, combos.data(), combos.size() * sizeof(DecodeCombine));
    if (!empty.empty()) memcpy(st + seg_bytes + combo_bytes, empty.data(), empty.size() * sizeof(int32_t));
    if (mfma_ok) {
        memcpy(st + base_total, mp.data(), mp.size() * sizeof(MfmaPiece));
        MfmaSlotHead* heads = reinterpret_cast<MfmaSlotHead*>(st + base_total + mp_bytes);
        for (size_t sl = 0; sl < nheads; ++sl) {
            const int32_t b0 = mptr[sl], e0 = mptr[sl + 1];
            MfmaSlotHead hd = {b0, e0, 0, 0, 0, 0, 0, 0, -1, 0, 0, 0, 0, {0, 0, 0}};
            if (b0 < e0) {
                const MfmaTile& r = mt[(size_t)b0];
                const MfmaPiece& pc = mp[(size_t)r.piece];
                hd.idx0 = r.idx0; hd.idx1 = r.idx1; hd.t = r.t;
                hd.seq = pc.seq; hd.kvh = pc.kvh;
                hd.flags = (r.t == pc.tile_begin ? 1 : 0) | (r.t + 1 == pc.tile_end ? 2 : 0);
                hd.partial = pc.partial; hd.tile_end = pc.tile_end; hd.seq_len = pc.seq_len; hd.kv_head = pc.kv_head;
                hd.piece = r.piece;
            }
            heads[sl] = hd;
        }
        if (!mc.empty()) memcpy(st + base_total + mp_bytes + mptr_bytes, mc.data(), mc.size() * sizeof(MfmaCombine));
        memcpy(st + base_total + mp_bytes + mptr_bytes + mc_bytes, mt.data(), mt.size() * sizeof(MfmaTile));
        if (units_ok && !p->h_units.empty()) memcpy(st + mfma_total, p->h_units.data(), p->h_units.size() * sizeof(MfmaUnit));
    }
    if (total) BZ_CHECK_HIP(hipMemcpyAsync(int_buffer, st, total, hipMemcpyHostToDevice, s));
    BZ_CHECK_HIP(hipEventRecord(p->upload_done, s));

    p->segments_d = (const DecodeSegment*)int_buffer;
    p->combos_d = (const DecodeCombine*)((char*)int_buffer + seg_bytes);
    p->empty_d = (const int32_t*)((char*)int_buffer + seg_bytes + combo_bytes);
    p->float_buffer_bytes = float_buffer_bytes;
    p->general_part_bytes = part_o_bytes + part_lse_bytes;
    p->max_seq_len = 0;
    for (uint32_t b = 0; b < batch_size; ++b) {
        const int32_t np = indptr_h[b + 1] - indptr_h[b];
        if (np > 0) p->max_seq_len = std::max<uint32_t>(p->max_seq_len, (uint32_t)(np - 1) * page_size + (uint32_t)last_page_len_h[b]);
    }
    p->part_o = (float*)float_buffer;
    p->part_lse = (float*)((char*)float_buffer + part_o_bytes);
    p->batch_size = batch_size; p->num_qo_heads = num_qo_heads; p->num_kv_heads = num_kv_heads;
    p->head_dim = head_dim; p->page_size = page_size;
    p->num_segments = (uint32_t)segs.size(); p->num_combos = (uint32_t)combos.size();
    p->num_empty = (uint32_t)empty.size(); p->num_partials = partials;
    p->num_workgroups = (uint32_t)segs.size() * num_kv_heads;
    p->mfma_ok = mfma_ok;
    if (mfma_ok) {
        p->mfma_pieces_d = (const MfmaPiece*)((char*)int_buffer + base_total);
        p->mfma_heads_d = (const MfmaSlotHead*)((char*)int_buffer + base_total + mp_bytes);
        p->mfma_combos_d = (const MfmaCombine*)((char*)int_buffer + base_total + mp_bytes + mptr_bytes);
        p->mfma_tiles_d = (const MfmaTile*)((char*)int_buffer + base_total + mp_bytes + mptr_bytes + mc_bytes);
        p->mfma_part_o = (float*)float_buffer; // the two paths never run in the same call: same workspace
        p->mfma_part_lse = (float*)((char*)float_buffer + mpart_o_bytes);
        p->mfma_units_d = units_ok ? (const MfmaUnit*)((char*)int_buffer + mfma_total) : nullptr;
        p->mfma_units = (uint32_t)p->h_units.size();
        p->mfma_unit_max_count = 0;
        for (const MfmaUnit& u : p->h_units) p->mfma_unit_max_count = std::max(p->mfma_unit_max_count, (uint32_t)u.count);
        p->mfma_slots = (uint32_t)mptr.size() - 1;
        p->mfma_pieces = (uint32_t)mp.size();
        p->mfma_combos = (uint32_t)mc.size();
        p->mfma_partials = mfma_partials;
        int32_t last = -1;
        p->mfma_split_seqs = 0;
        p->mfma_max_count = 0;
        for (const MfmaCombine& c : mc) {
            if (c.seq != last) { ++p->mfma_split_seqs; last = c.seq; }
            p->mfma_max_count = std::max(p->mfma_max_count, (uint32_t)c.count);
        }
    }
    // BZ_DECODE_PATH=general keeps the MFMA kernel out (used to test the general kernel on shapes
    // both kernels cover); BZ_DECODE_PATH=one_call makes the decode step take its one-call form wherever
    // it applies, also where the two calls are the faster choice (used to test it on such batches)
    const char* path = getenv("BZ_DECODE_PATH");
    p->force_general = path && !strcmp(path, "general");
    const bool force_one_call = path && !strcmp(path, "one_call");

    // Form of the decode step.  In its one-call form every piece goes through a partial row that the
    // finishing kernel reads back; in the two calls a (sequence, kv head) that one wave slot holds whole
    // writes its final rows at once.  So the one call pays where most of them are split over wave slots
    // anyway (batches with fewer of them than the launch has slots), and the two calls are taken where most
    // are whole (1024 sequences of 64 tokens: 63 us against 77 us).  The one call also needs room for one
    // partial per piece in the float workspace.
    {
        const size_t part_o_bytes = ((size_t)p->mfma_pieces * 16 * 128 * sizeof(float) + 255) / 256 * 256;
        const size_t part_lse_bytes = ((size_t)p->mfma_pieces * 16 * sizeof(float) + 255) / 256 * 256;
        const bool applies = p->mfma_ok && !p->force_general && p->mfma_slots > 0 && p->mfma_units_d &&
                             p->mfma_units > 0 && part_o_bytes + part_lse_bytes <= p->float_buffer_bytes;
        const bool mostly_split = 2 * (uint64_t)p->mfma_combos >= p->mfma_units;
        p->step_one_call = applies && (force_one_call || mostly_split);
    }

    (void)decode_noalloc_prepare(); // (a failure is reported by bz_batch_decode_noalloc itself, should it be called)
    p->planned = true;
    return 0;
}

extern "C" int bz_decode_plan_workspace(bz_decode_plan_t* plan_, const int32_t* indptr_h, const int32_t* last_page_len_h,
                                        uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads,
                                        uint32_t head_dim, uint32_t page_size, uint32_t split_tokens,
                                        uint32_t num_compute_units, size_t* float_buffer_bytes,
                                        size_t* int_buffer_bytes) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p || !indptr_h || !last_page_len_h) return BZ_ERR_BAD_ARG;
    if (page_size == 0 || num_kv_heads == 0 || num_qo_heads % num_kv_heads) return BZ_ERR_BAD_ARG;
    p->planned = false; // the host scratch no longer matches what the device holds
    ScheduleCounts counts;
    const int cus = num_compute_units ? (int)num_compute_units : device_cu_count();
    const int rc = build_schedule(p, indptr_h, last_page_len_h, batch_size, num_qo_heads, num_kv_heads, head_dim,
                                  page_size, split_tokens, cus, &counts);
    if (rc) return rc;
    const ScheduleLayout L = schedule_layout(p, counts, num_qo_heads, head_dim);
    const bool mfma = counts.mfma_shape && !p->h_pieces.empty();
    // (the one-call decode step keeps one partial per piece, split or not, and reads the unit list)
    if (float_buffer_bytes)
        *float_buffer_bytes = std::max(L.part_o_bytes + L.part_lse_bytes,
                                       mfma ? std::max(L.mpart_o_bytes + L.mpart_lse_bytes,
                                                       L.step_part_o_bytes + L.step_part_lse_bytes) : 0);
    if (int_buffer_bytes)
        *int_buffer_bytes = L.base_total + (mfma ? L.mp_bytes + L.mptr_bytes + L.mc_bytes + L.cnt_bytes + L.unit_bytes : 0);
    return 0;
}

extern "C" int bz_decode_plan_host_schedule(const bz_decode_plan_t* plan_, int which, const int32_t** data,
                                            size_t* num_records, uint32_t* ints_per_record) {
    const DecodePlan* p = reinterpret_cast<const DecodePlan*>(plan_);
    if (!p || !data || !num_records || !ints_per_record) return BZ_ERR_BAD_ARG;
    switch (which) {
    case 0: *data = (const int32_t*)p->h_segs.data(); *num_records = p->h_segs.size(); *ints_per_record = sizeof(DecodeSegment) / 4; break;
    case 1: *data = (const int32_t*)p->h_combos.data(); *num_records = p->h_combos.size(); *ints_per_record = sizeof(DecodeCombine) / 4; break;
    case 2: *data = p->h_empty.data(); *num_records = p->h_empty.size(); *ints_per_record = 1; break;
    case 3: *data = (const int32_t*)p->h_tiles.data(); *num_records = p->h_tiles.size(); *ints_per_record = sizeof(MfmaTile) / 4; break;
    case 4: *data = p->h_slot_ptr.data(); *num_records = p->h_slot_ptr.size(); *ints_per_record = 1; break;
    case 5: *data = (const int32_t*)p->h_pieces.data(); *num_records = p->h_pieces.size(); *ints_per_record = sizeof(MfmaPiece) / 4; break;
    case 6: *data = (const int32_t*)p->h_mcombos.data(); *num_records = p->h_mcombos.size(); *ints_per_record = sizeof(MfmaCombine) / 4; break;
    case 7: *data = (const int32_t*)p->h_units.data(); *num_records = p->h_units.size(); *ints_per_record = sizeof(MfmaUnit) / 4; break;
    default: return BZ_ERR_BAD_ARG;
    }
    return 0;
}

extern "C" int bz_decode_plan_info(const bz_decode_plan_t* plan_, uint32_t* num_segments, uint32_t* num_split_seqs,
                                   uint32_t* num_workgroups) {
    const DecodePlan* p = reinterpret_cast<const DecodePlan*>(plan_);
    if (!p || !p->planned) return BZ_ERR_NOT_PLANNED;
    const bool mfma = p->mfma_ok && !p->force_general;
    if (num_segments) *num_segments = mfma ? p->mfma_pieces : p->num_segments;
    if (num_split_seqs) *num_split_seqs = mfma ? p->mfma_split_seqs : p->num_combos;
    if (num_workgroups) *num_workgroups = mfma ? p->mfma_slots : p->num_workgroups;
    return 0;
}

extern "C" int bz_decode_plan_step_form(const bz_decode_plan_t* plan_) {
    const DecodePlan* p = reinterpret_cast<const DecodePlan*>(plan_);
    if (!p || !p->planned) return BZ_ERR_NOT_PLANNED;
    return p->step_one_call ? 1 : 0;
}

extern "C" int bz_decode_plan_set_timing_events(bz_decode_plan_t* plan_, void* start_event, void* stop_event) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p || ((start_event == nullptr) != (stop_event == nullptr))) return BZ_ERR_BAD_ARG;
    p->time_start = (hipEvent_t)start_event;
    p->time_stop = (hipEvent_t)stop_event;
    return 0;
}
