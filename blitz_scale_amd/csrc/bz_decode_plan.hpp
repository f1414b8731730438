// Decode schedule shared by the host planner and the decode kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <new>
#include <vector>

namespace bz {

// One contiguous, page-aligned piece of one sequence's context.
struct DecodeSegment {
    int32_t seq;        // sequence index b
    int32_t page_begin; // first page of the piece, relative to indptr[b]
    int32_t page_end;   // one past the last page, relative to indptr[b]
    int32_t partial;    // -1: the piece is the whole sequence, write the final row;
                        // >=0: slot of the split-K partial result in the float workspace
};

// One split sequence: its partials are slots [first, first+count).
struct DecodeCombine {
    int32_t seq, first, count, pad;
};

// MFMA path: a contiguous run of 32-token tiles of one (sequence, kv head).
struct MfmaPiece {
    int32_t seq, kvh;
    int32_t tile_begin, tile_end; // in 32-token tiles from the start of the sequence
    int32_t partial;              // -1: whole (sequence, kv head) -> final rows; else partial slot
    int32_t combo, count, first;  // split (sequence, kv head): its index, number of partials, first slot
    int32_t ip0, npages, seq_len; // indptr[seq], pages and tokens of the sequence (from the host table)
    int32_t kv_head;              // the kv head whose K/V the piece reads (kvh above is the scheduled unit:
                                  // kv_head * parts + part when a kv head has more than 16 q heads)
    int32_t pad[4];
};

// One 32-token tile of a wave slot's share, in processing order.
struct MfmaTile {
    int32_t idx0, idx1; // positions in indices[] of the pages of the two 16-token subtiles (kept in range)
    int32_t t;          // tile number inside its sequence
    int32_t piece;      // index into the piece array
};

// What a wave slot reads first: its range of tile records and the full description of the first of
// them (record and piece joined), so that the loads of the first tile go out after one round trip.
struct MfmaSlotHead {
    int32_t begin, end;   // tile records [begin, end)
    int32_t idx0, idx1, t; // the first record
    int32_t seq, kvh;
    int32_t flags;        // 1: first tile of its piece, 2: last tile of its piece
    int32_t partial;      // -1 or partial slot
    int32_t tile_end;     // one past the last tile of the piece
    int32_t seq_len;
    int32_t kv_head;      // kv head of the first tile's piece
    int32_t piece;        // index of the first tile's piece (its partial slot in the one-call decode step)
    int32_t pad[3];
};

// One (sequence, scheduled kv-head unit) with its pieces, for the finishing kernel of the one-call decode
// step: pieces [first_piece, first_piece + count) are consecutive, and in that mode piece i writes partial
// slot i.
struct MfmaUnit {
    int32_t seq, unit, first_piece, count;
    int32_t ip0, seq_len; // indptr[seq] and the tokens of the sequence, from the host table the plan was made from
    int32_t pad[2]; // zero (the finishing kernel reads pad[0] where the caller has no step counter)
};

// Growable array of plain records that does not clear what it hands out (the planner overwrites every
// record it counts).
template <typename T> struct RawArray {
    T* ptr = nullptr;
    size_t n = 0, cap = 0;
    RawArray() = default;
    RawArray(const RawArray&) = delete;
    RawArray& operator=(const RawArray&) = delete;
    ~RawArray() { ::operator delete(ptr); }
    void resize_uninitialized(size_t count) {
        if (count > cap) {
            ::operator delete(ptr);
            cap = count + count / 2 + 64;
            ptr = static_cast<T*>(::operator new(cap * sizeof(T)));
        }
        n = count;
    }
    void clear() { n = 0; }
    size_t size() const { return n; }
    bool empty() const { return n == 0; }
    T* data() { return ptr; }
    const T* data() const { return ptr; }
    T& operator[](size_t i) { return ptr[i]; }
    const T& operator[](size_t i) const { return ptr[i]; }
};

// One split (sequence, kv head): partial slots [first, first+count).
struct MfmaCombine {
    int32_t seq, kvh, first, count;
};

struct DecodePlan {
    bool planned = false;
    uint32_t batch_size = 0, num_qo_heads = 0, num_kv_heads = 0, head_dim = 0, page_size = 0;
    uint32_t num_segments = 0, num_combos = 0, num_empty = 0, num_partials = 0;
    uint32_t num_workgroups = 0;
    // device views into the caller's workspaces
    const DecodeSegment* segments_d = nullptr;
    const DecodeCombine* combos_d = nullptr;
    const int32_t* empty_d = nullptr;
    float* part_o = nullptr;
    float* part_lse = nullptr;
    // MFMA path schedule (valid when mfma_ok)
    bool mfma_ok = false;
    bool force_general = false; // tests: run the general kernel even where the MFMA path applies
    bool step_one_call = false;  // bz_decode_step runs its two-launch form (else the append and the decode calls)
    uint32_t mfma_slots = 0, mfma_combos = 0, mfma_partials = 0, mfma_pieces = 0, mfma_split_seqs = 0;
    uint32_t mfma_max_count = 0; // most partials any split (sequence, kv head) has
    bool mfma_streaming = false; // every wave slot has two tiles or more (bandwidth-bound launch)
    uint32_t mfma_parts = 1;     // groups of more than 16 q heads are scheduled as this many equal parts per kv head
    const MfmaPiece* mfma_pieces_d = nullptr;
    const MfmaCombine* mfma_combos_d = nullptr;
    const MfmaTile* mfma_tiles_d = nullptr;
    const MfmaSlotHead* mfma_heads_d = nullptr; // one per wave slot
    const MfmaUnit* mfma_units_d = nullptr;     // every (sequence with pages, unit); nullptr when it did not fit
    uint32_t mfma_units = 0;
    uint32_t mfma_unit_max_count = 0;           // most pieces any (sequence, unit) has
    size_t float_buffer_bytes = 0;              // size of the float workspace given to plan()
    float* mfma_part_o = nullptr;
    float* mfma_part_lse = nullptr;
    // general kernel, BZ_ROPE_FULL: (cos, sin) of position * frequency for every position of the planned table,
    // kept in the float workspace behind the general kernel's partials and filled by the first such call after
    // a plan() (any call that puts matrix-core partials into the workspace invalidates it)
    uint32_t max_seq_len = 0;       // longest sequence of the planned table
    size_t general_part_bytes = 0;  // bytes of the general kernel's partials at the start of the float workspace
    // host scratch of plan(), kept between calls so that a step's plan neither allocates nor faults in
    // fresh pages (the schedule of a large batch is around a megabyte)
    std::vector<DecodeSegment> h_segs;
    std::vector<DecodeCombine> h_combos;
    std::vector<int32_t> h_empty, h_slot_ptr;
    std::vector<MfmaPiece> h_pieces;
    RawArray<MfmaTile> h_tiles;
    std::vector<MfmaCombine> h_mcombos;
    std::vector<MfmaUnit> h_units;
    // pinned staging for the schedule upload and the event that guards its reuse
    void* staging = nullptr;
    size_t staging_bytes = 0;
    hipEvent_t upload_done = nullptr;
    hipEvent_t time_start = nullptr, time_stop = nullptr; // optional: bracket the decode kernel launch
    int device = -1;
};

// Looks up, for the current device, the address of the fixed array that bz_batch_decode_noalloc keeps its
// partial results in (bz_decode.hip); called by bz_decode_plan so that the call itself only launches kernels.
int decode_noalloc_prepare();

} // namespace bz
