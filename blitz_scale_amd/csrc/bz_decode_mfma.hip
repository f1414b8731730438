// MFMA paged decode for gfx950 (head_dim 128, page_size a multiple of 16, f16/bf16/e4m3 KV, up to 16
// query heads per scheduled unit; the planner cuts a larger group into equal parts).  One wave64 per
// workgroup walks a list of "pieces" (contiguous runs of 32-token tiles of one (sequence, kv head)) that
// the host planner balanced over the wave slots of the chip, so every K and V byte is read once and
// shared by all query heads of the group.
//
// Per 32-token tile, with S^T = K Q^T so that the MFMA result layout of the scores is already the
// A-operand layout of the P V product (no shuffles between the two contractions):
//   K rows   : global -> VGPR, 16 B per lane, used directly as MFMA A operands (contraction over d)
//   V rows   : global -> VGPR -> LDS (row stride 288 B), read back with the transposing LDS load
//              (ds_read_b64_tr_b16) as MFMA B operands (contraction over tokens)
//   softmax  : online, 8 scores per lane, row max / sum over the 4 lane groups with two shuffles
// The loads of tile t+1 are issued before the arithmetic of tile t; with one-byte pools, whose tiles need half
// the landing registers, two tiles are in flight per wave.  The rows of a finished piece wait in LDS and are
// stored when the wave slot is done: between its first load and its last tile a wave issues no store.
#include <cmath>
#include <type_traits>

#include "bz_common.hpp"
#include "bz_decode_plan.hpp"

namespace bz {

// K and V are read exactly once per launch, so their loads carry the non-temporal hint (the lines are
// not kept in L2 / MALL for a second use that never comes).  Measured on 128 sequences x 32/8 heads,
// bf16: 120.6 -> 110.3 us with the hint on K and V, 110.6 us on V alone, 118.4 us on K alone.  V loads
// cover whole 128-byte lines; K loads cover half a line per instruction, and for one-byte pools the
// hint on K costs 6 % (429 against 403 us at 256 x 4096 tokens) while the hint on V alone gains 2 %,
// so one-byte pools keep plain K loads.  Mixing hinted and plain loads on the halves of one line is
// worse than either (117.8 us).  A launch in which a wave slot has a single tile is bound by latency, not by
// bandwidth, and runs 1.5 to 2 us slower with the hint (8 sequences x 1024 tokens: 14.1 -> 15.8 us), so
// the planner switches the hint on (template parameter NT) only when every slot loops over two tiles or
// more.  (Chosen per load by a wave-uniform run-time flag instead, the kernel ran six times slower.)
#ifndef BZ_NT_MASK // build knob for A/B measurements: 1 = K of 16-bit pools, 8 = V of 16-bit pools, 4 / 2 = K / V of one-byte pools
#define BZ_NT_MASK 11
#endif
constexpr bool kNtK16 = (BZ_NT_MASK & 1) != 0, kNtV16 = (BZ_NT_MASK & 8) != 0, kNtK8 = (BZ_NT_MASK & 4) != 0,
               kNtV8 = (BZ_NT_MASK & 2) != 0;
typedef unsigned int bz_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld_kv16(const char* p, bool nt) {
    if (nt) {
        const bz_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const bz_u32x4_t*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    } else {
        return *reinterpret_cast<const uint4*>(p);
    }
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;

constexpr int kTileTok = 32;     // tokens per tile
constexpr int kVRowBytes = 288;  // LDS row stride of the V tile: 256 B of data + 32 B so that
                                 // consecutive rows start 8 banks apart (conflict-free transposed reads)

struct MfmaDecodeArgs {
    const void* q;
    void* out;
    float* lse;
    const char* k_data;
    const char* v_data;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    const int32_t* steps_ahead; // optional: the table (and the plan made from it) is this many steps ahead
    const MfmaPiece* pieces;
    const MfmaTile* tiles;
    const MfmaSlotHead* heads;
    float* part_o;   // [num_partials][16][128]
    float* part_lse; // [num_partials][16]
    uint64_t stride_page, stride_n, stride_h; // elements
    uint32_t page_size, num_qo_heads, group; // group: q heads per scheduled unit (<= 16)
    int rope_q;
    int step_mode; // 1 = first half of the one-call decode step: the last token of every sequence is left to the
                   // finishing kernel (which also appends it), q is rotated at its position, and every piece,
                   // split or not, leaves a partial result in the slot numbered like the piece
    float sm_scale_log2;
    const float* k_scale; // e4m3 pool only: per-kv-head dequantisation factors (nullptr = 1)
    const float* v_scale;
    RopeFreqs freqs;
};

template <bool BF16> struct Mma;
template <> struct Mma<true> {
    using vec = bf16x8_t;
    __device__ static __forceinline__ f32x4_t run(uint4 a, uint4 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                       c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        return f32x2_to_bf16x2_bits(lo, hi);
    }
    __device__ static __forceinline__ float unpack_lo(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static __forceinline__ float unpack_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};
template <> struct Mma<false> {
    using vec = f16x8_t;
    __device__ static __forceinline__ f32x4_t run(uint4 a, uint4 b, f32x4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                      0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        return (uint32_t)f32_to_f16_bits(lo) | ((uint32_t)f32_to_f16_bits(hi) << 16);
    }
    __device__ static __forceinline__ float unpack_lo(uint32_t w) {
        return __half2float(__ushort_as_half((uint16_t)(w & 0xffffu)));
    }
    __device__ static __forceinline__ float unpack_hi(uint32_t w) {
        return __half2float(__ushort_as_half((uint16_t)(w >> 16)));
    }
};

__device__ __forceinline__ uint32_t& u4(uint4& v, int i) { return reinterpret_cast<uint32_t*>(&v)[i]; }

// Four OCP e4m3 bytes -> four values of the 16-bit MFMA operand type.  Every e4m3 value is exactly
// representable in f16 and in bf16; gfx950 converts a pair of bytes straight to a pair of 16-bit values
// (v_cvt_scalef32_pk_{bf16,f16}_fp8 with a unit scale), half the instructions of the way through fp32.
typedef __attribute__((ext_vector_type(2))) __bf16 mfma_bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 mfma_f16x2_t;
template <bool BF16> __device__ __forceinline__ uint2 fp8x4_to_op(uint32_t w) {
    if constexpr (BF16) {
        const mfma_bf16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
        const mfma_bf16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
        return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
    } else {
        const mfma_f16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
        const mfma_f16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
        return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
    }
}
// bytes 8e .. 8e+7 of a 16-byte register -> one 8-element MFMA operand
template <bool BF16> __device__ __forceinline__ uint4 fp8x8_to_op(const uint4& r, int e) {
    const uint32_t w0 = e ? r.z : r.x, w1 = e ? r.w : r.y;
    const uint2 a = fp8x4_to_op<BF16>(w0), b = fp8x4_to_op<BF16>(w1);
    return make_uint4(a.x, a.y, b.x, b.y);
}

// The read-only inputs are separate __restrict__ parameters so that wave-uniform reads go through
// the scalar unit.
//
// Under load a dependent memory round trip costs several microseconds, so the kernel has none in its
// steady state: the planner lists every tile of a wave slot as a 16-byte record, and the wave fetches
// the records, the page ids they point at and the metadata of their pieces for 16 tiles at a time
// (one lane per tile) well before they are needed; inside the tile loop everything wave-uniform comes
// out of those registers with v_readlane.  The K/V loads of tile g+1 and the q rows of the next piece
// are issued before the arithmetic of tile g.
// wave-level ordering of LDS traffic: LDS instructions of one wave execute in order, so making the
// compiler keep the order is all that is needed (a workgroup barrier would also drain the global loads
// that are in flight for the next tile)
// 16 bytes to global memory through a pointer whose address space the compiler cannot see (it came out of LDS):
// said explicitly, so that the store is a global one and not a flat one, which would also count as an LDS access.
__device__ __forceinline__ void store_global_16(void* p, float a, float b, float c, float d) {
    typedef float vec4 __attribute__((ext_vector_type(4)));
    *(__attribute__((address_space(1))) vec4*)p = vec4{a, b, c, d};
}

__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kInfoInts = 12; // per-tile description kept in LDS (see fetch_info): 10 ints, padded
constexpr int kInfoChunk = 16; // tile descriptions fetched per round trip (one lane per tile)

// (Measured and not kept: K rows fetched like V -- four whole 256-byte rows per wave instruction, so that the
// non-temporal hint covers whole 128-byte lines -- parked in LDS with an XOR swizzle and read back in the
// A-operand layout.  Same results, but 125 us against 109 us on 128 sequences x 32/8 heads bf16 and 234 against
// 208 us on 64 x 32/32 heads: the extra LDS round trip sits between a tile's arrival and its arithmetic.)

// KV8: the pool holds e4m3 bytes.  K and V are widened to the 16-bit type of q in registers (exactly)
// on their way to the matrix cores; the per-head scales are folded into the softmax scale and into
// the final normalisation.  A lane then fetches 16 bytes = 16 elements of a K row, so the contraction
// index of MFMA step ks, lane group j, element i is d = 64*(ks/2) + 16*j + 8*(ks%2) + i (q follows).
// NT: K/V loads carry the non-temporal hint (see kNtK16 above); chosen by the planner.
template <bool BF16, typename OT, bool ROPE_Q, bool KV8, bool NT>
__global__ __launch_bounds__(64, 2) void decode_mfma_kernel(const MfmaSlotHead* __restrict__ heads, MfmaDecodeArgs a,
                                                            const char* __restrict__ q_ptr,
                                                            const char* __restrict__ k_data,
                                                            const char* __restrict__ v_data,
                                                            const int32_t* __restrict__ indices,
                                                            const MfmaPiece* __restrict__ pieces,
                                                            const MfmaTile* __restrict__ tiles,
                                                            const float* __restrict__ k_scale,
                                                            const float* __restrict__ v_scale) {
    using M = Mma<BF16>;
    __shared__ __attribute__((aligned(16))) unsigned char v_lds[kTileTok * kVRowBytes];
    __shared__ __attribute__((aligned(16))) int info_lds[2][kInfoChunk][kInfoInts];
    // Normalised rows of finished pieces, kept here until the slot's last tile is done (or the space runs out):
    // 16 rows of 128 floats (+ 4 per row, so that the four lane groups fall on different banks), one log-sum-exp
    // per row, and for each parked piece where its rows go.
    constexpr int kStageRow = 132, kStageRows = 16, kStagePieces = 8;
    struct StagedPiece { char* dst; float* lse; int row0, rows, f32, pad; };
    __shared__ __attribute__((aligned(16))) float stage_lds[kStageRows * kStageRow + kStageRows];
    __shared__ StagedPiece stage_desc[kStagePieces];

    // cos / sin of position * frequency i for the piece being opened: one sincosf per lane instead of
    // sixteen (each lane needs the angles of its own 16 contraction indices)
    __shared__ float rope_cs[ROPE_Q ? 2 : 1][64];

    const int lane = threadIdx.x;
    const int n = lane & 15; // query head (scores) / d column (output) / token row (K operand)
    const int j = lane >> 4; // lane group: which 8-wide slice of the MFMA contraction
    const int P = (int)a.page_size;
    constexpr int ES = KV8 ? 1 : 2; // bytes per pool element
    const size_t row_bytes = (size_t)a.stride_n * ES;
    auto d_of = [&](int ks) { return KV8 ? 64 * (ks >> 1) + 16 * j + 8 * (ks & 1) : 32 * ks + 8 * j; };
    const int G = (int)a.group;

    // A plan made from a table that runs ahead lists tiles up to the future lengths; at present every
    // sequence is `ahead` tokens shorter.  Tiles past the present end are masked as a whole (their pages
    // exist), so a piece can come out empty: zero weight in the split-K combine.
    // The slot's head holds its range of tile records and the description of the first tile: after one
    // round trip (head and counter together) only the two page ids stand between the wave and its first
    // K/V loads.
    // (`heads` is the kernel's first argument: with the kernel-argument preload the build asks for it arrives in
    // registers with the wave, and the slot head is asked for together with the other arguments, not behind them)
    const MfmaSlotHead* __restrict__ head = heads + blockIdx.x;
    const int g_begin = head->begin, g_end = head->end;
    const MfmaSlotHead first = *head;
    // This lane's rotation frequency, fetched once and here, beside the scalar loads of the slot head: read where a
    // piece is opened, the load would sit behind the tile's K/V loads in the (in-order) queue, and the angles and
    // the rotation of q -- some 400 instructions -- would start only after the tile has arrived instead of running
    // while it travels.
    float lane_freq = 0.f;
    if (ROPE_Q) {
        lane_freq = a.freqs.f[lane];
        asm("" : "+v"(lane_freq)); // (kept in its register: not fetched again at the point of use)
    }
    // Left to the compiler, the slot head is fetched in two steps (its tile range, then, behind the test for an empty
    // slot, the rest together with most of the kernel's arguments): one more scalar round trip in front of the first
    // page ids.  The empty asm below needs a value made of all of them, so they are all asked for here, in one batch.
    uint32_t early = (uint32_t)first.idx0 ^ (uint32_t)first.idx1 ^ (uint32_t)first.t ^ (uint32_t)first.seq ^ (uint32_t)first.kvh ^
                     (uint32_t)first.flags ^ (uint32_t)first.partial ^ (uint32_t)first.tile_end ^ (uint32_t)first.seq_len ^
                     (uint32_t)first.kv_head ^ (uint32_t)first.piece;
    early ^= (uint32_t)(uintptr_t)a.steps_ahead ^ (uint32_t)(uintptr_t)tiles ^ (uint32_t)(uintptr_t)indices ^ (uint32_t)(uintptr_t)pieces ^ (uint32_t)(uintptr_t)k_data ^
             (uint32_t)(uintptr_t)v_data ^ (uint32_t)(uintptr_t)q_ptr;
    early ^= (uint32_t)a.stride_page ^ (uint32_t)a.stride_n ^ (uint32_t)a.stride_h ^ a.page_size ^ a.num_qo_heads ^ a.group ^
             (uint32_t)a.step_mode;
    asm("" : "+s"(early));
    // (g_begin is never negative: the second term only keeps the value above in use)
    if (g_begin >= g_end || (g_begin < 0 && early == 0x9e3779b9u)) return;
    int first_pid0 = indices[first.idx0], first_pid1 = indices[first.idx1];
    const int ahead_raw = a.steps_ahead ? *a.steps_ahead : 0; // (beside the page ids: the same round trip)
    const int ahead = max(ahead_raw, 0);

    // ---- descriptions of kInfoChunk tiles at a time: lane l < kInfoChunk fetches the record of tile base+l, the two
    // page ids it points at and the piece it belongs to, and leaves 10 ints in LDS:
    //   [pid0, pid1, t, seq | kvh, flags (1: first tile of its piece, 2: last), partial, tok_end | seq_len, kv head]
    struct Desc { int v[10]; };
    // (in three steps, so that the prologue can put other loads between them: the record, what the record points at,
    // and the arithmetic on both)
    struct InfoRaw { int4 m0, m1, m2; int pid0, pid1; };
    // (lanes past the slot's last tile fetch that tile once more: loads under a lane mask would make the compiler
    // wait for them on the spot, before it zeroes the other lanes' registers)
    auto fetch_rec = [&](int base) -> MfmaTile { return tiles[min(base + (lane & (kInfoChunk - 1)), g_end - 1)]; };
    auto fetch_dep = [&](const MfmaTile& rec) -> InfoRaw {
        InfoRaw r;
        r.m0 = *reinterpret_cast<const int4*>(&pieces[rec.piece]);
        r.m1 = *(reinterpret_cast<const int4*>(&pieces[rec.piece]) + 1);
        r.m2 = *(reinterpret_cast<const int4*>(&pieces[rec.piece]) + 2);
        r.pid0 = indices[rec.idx0];
        r.pid1 = indices[rec.idx1];
        return r;
    };
    auto make_desc = [&](const MfmaTile& rec, const InfoRaw& r) -> Desc {
        Desc d;
        d.v[0] = r.pid0;
        d.v[1] = r.pid1;
        d.v[2] = rec.t;
        d.v[3] = r.m0.x;                                           // seq
        d.v[4] = r.m0.y;                                           // kvh
        d.v[5] = (rec.t == r.m0.z ? 1 : 0) | (rec.t + 1 == r.m0.w ? 2 : 0);
        d.v[6] = a.step_mode ? rec.piece : r.m1.x;                 // partial slot or -1
        d.v[8] = max(r.m2.z - ahead - a.step_mode, 0);             // tokens attended over at present
        d.v[7] = min(r.m0.w * kTileTok, d.v[8]);                   // tok_end of the piece
        d.v[9] = r.m2.w;                                           // kv head whose K/V are read (kvh is the scheduled unit)
        return d;
    };
    auto fetch_info = [&](int base) -> Desc {
        const MfmaTile rec = fetch_rec(base);
        return make_desc(rec, fetch_dep(rec));
    };
    auto stash_info = [&](const Desc& d, int buf) {
        if (lane < kInfoChunk) {
            int* dst = &info_lds[buf][lane][0];
            *reinterpret_cast<int4*>(dst) = make_int4(d.v[0], d.v[1], d.v[2], d.v[3]);
            *reinterpret_cast<int4*>(dst + 4) = make_int4(d.v[4], d.v[5], d.v[6], d.v[7]);
            *reinterpret_cast<int2*>(dst + 8) = make_int2(d.v[8], d.v[9]);
        }
    };
    struct TileUni { int pid0, pid1, t, seq, kvh, flags, partial, tok_end, seq_len, kvr; }; // wave-uniform
    auto read_info = [&](int buf, int i) -> TileUni {
        const int* src = &info_lds[buf][i][0];
        const int4 x = *reinterpret_cast<const int4*>(src);
        const int4 y = *reinterpret_cast<const int4*>(src + 4);
        const int2 z2 = *reinterpret_cast<const int2*>(src + 8);
        const int z = z2.x;
        TileUni u;
        u.pid0 = __builtin_amdgcn_readfirstlane(x.x); u.pid1 = __builtin_amdgcn_readfirstlane(x.y);
        u.t = __builtin_amdgcn_readfirstlane(x.z); u.seq = __builtin_amdgcn_readfirstlane(x.w);
        u.kvh = __builtin_amdgcn_readfirstlane(y.x); u.flags = __builtin_amdgcn_readfirstlane(y.y);
        u.partial = __builtin_amdgcn_readfirstlane(y.z); u.tok_end = __builtin_amdgcn_readfirstlane(y.w);
        u.seq_len = __builtin_amdgcn_readfirstlane(z);
        u.kvr = __builtin_amdgcn_readfirstlane(z2.y);
        return u;
    };

    uint4 kreg[2][4], vreg[8], qnext[4];
    // byte offsets of the two 16-token subtiles of a tile inside the pool
    struct TileBase { size_t b[2]; };
    auto tile_base = [&](const TileUni& u) -> TileBase {
        TileBase r;
        const int pid[2] = {u.pid0, u.pid1};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int slot0 = (u.t * kTileTok + 16 * s) % P; // a subtile past the last page reads the last page, masked later
            r.b[s] = ((size_t)pid[s] * a.stride_page + (size_t)slot0 * a.stride_n + (size_t)u.kvr * a.stride_h) * ES;
        }
        return r;
    };
    // One-byte pools: a tile is 8 KiB and lands in half of the registers a 16-bit tile needs, so the two halves
    // are two sets (SET 0 / 1: kreg[u][2 SET + p], vreg[4 SET + w]) and two tiles are in flight per wave.
    // `live` false: the set has no tile to fetch; the loads are issued all the same, every lane at the tile's first
    // bytes (one cache line), so that the number of loads behind a set's own does not depend on the path taken
    // and the waits the compiler derives for the sets stay apart.
    auto issue_loads_kv8 = [&](const TileBase& tb, auto set_c, bool live) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_c)::value;
        const size_t base[2] = {tb.b[0], tb.b[1]};
        const size_t koff = live ? (size_t)n * row_bytes + (size_t)(j * 16) : 0;
#pragma unroll
        for (int p = 0; p < 2; ++p) { // 16 bytes feed MFMA steps 2p and 2p+1
            kreg[0][2 * SET + p] = ld_kv16(k_data + base[0] + koff + (live ? p * 64 : 0), NT && kNtK8);
            kreg[1][2 * SET + p] = ld_kv16(k_data + base[1] + koff + (live ? p * 64 : 0), NT && kNtK8);
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) { // rows 8w..8w+7 of the tile, 8 lanes x 16 B per 128-byte row
            const int row = 8 * w + (lane >> 3);
            const size_t voff = live ? (size_t)(row & 15) * row_bytes + (size_t)((lane & 7) * 16) : 0;
            vreg[4 * SET + w] = ld_kv16(v_data + base[live ? (row >> 4) : 0] + voff, NT && kNtV8);
        }
    };
    auto issue_loads = [&](const TileBase& tb) {
        const size_t base[2] = {tb.b[0], tb.b[1]};
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            kreg[0][ks] = ld_kv16(k_data + base[0] + (size_t)n * row_bytes + ks * 64 + j * 16, NT && kNtK16);
            kreg[1][ks] = ld_kv16(k_data + base[1] + (size_t)n * row_bytes + ks * 64 + j * 16, NT && kNtK16);
        }
#pragma unroll
        for (int w = 0; w < 8; ++w) { // rows 4w..4w+3 of the tile, 16 lanes x 16 B per row
            const int row = 4 * w + j;
            vreg[w] = ld_kv16(v_data + base[row >> 4] + (size_t)(row & 15) * row_bytes + n * 16, NT && kNtV16);
        }
    };
    // q rows of a piece as MFMA B operand: lane (head n, group j) holds q[head][32*ks + 8*j .. +7]
    // (every lane loads: columns past the group fetch its last head again and are zeroed where the piece is opened --
    // loads under a lane mask would make the compiler wait for them on the spot)
    auto issue_q = [&](const TileUni& u) {
        const char* qrow = q_ptr + ((size_t)u.seq * a.num_qo_heads + (size_t)u.kvh * G + min(n, G - 1)) * 256;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qnext[ks] = *reinterpret_cast<const uint4*>(qrow + d_of(ks) * 2);
    };

    // The records of the first tiles are requested together with the two page ids of the first tile (whose
    // description came with the slot head); what the records point at -- pieces, page ids -- goes out as soon as both
    // are there, and the first tile's q, K and V right behind it, so that the records are turned into descriptions
    // and parked in LDS while the first tile travels.  (With the whole fetch in front, its second round trip stood
    // between the slot head and the first K/V loads.  A slot with a single tile -- small batches -- needs no records.)
    const bool multi = g_end - g_begin > 1;
    TileUni un; // description of the tile whose loads are issued next
    un.pid0 = first_pid0;
    un.pid1 = first_pid1;
    MfmaTile rec0 = {0, 0, 0, 0};
    if (multi) rec0 = fetch_rec(g_begin);
    asm("" : "+s"(un.pid0), "+s"(un.pid1)); // (asked for here, beside the records, not where the addresses are formed)
    un.t = first.t; un.seq = first.seq; un.kvh = first.kvh; un.flags = first.flags;
    un.partial = a.step_mode ? first.piece : first.partial;
    un.kvr = first.kv_head;
    un.seq_len = max(first.seq_len - ahead - a.step_mode, 0);
    un.tok_end = min(first.tile_end * kTileTok, un.seq_len);
    __builtin_amdgcn_sched_barrier(0);
    InfoRaw raw0 = {};
    if (multi) raw0 = fetch_dep(rec0);
    __builtin_amdgcn_sched_barrier(0);
    issue_q(un);
    if constexpr (KV8) issue_loads_kv8(tile_base(un), std::integral_constant<int, 0>{}, true);
    else issue_loads(tile_base(un));
    __builtin_amdgcn_sched_barrier(0);
    if (multi) {
        stash_info(make_desc(rec0, raw0), 0);
        wave_lds_sync();
    }
    int chunk_base = g_begin, buf = 0;
    Desc dnext;

    uint4 qhi[4], qlo[4];
    float m_run = -INFINITY, l_run = 0.f;
    f32x4_t acc[8];

    // descriptions of the next chunk of tiles: fetched a quarter into this chunk, parked in the other LDS
    // buffer at three quarters
    auto info_traffic = [&](int i) __attribute__((always_inline)) {
        if (i == kInfoChunk / 4 && chunk_base + kInfoChunk < g_end) dnext = fetch_info(chunk_base + kInfoChunk);
        if (i == 3 * kInfoChunk / 4 && chunk_base + kInfoChunk < g_end) { stash_info(dnext, buf ^ 1); wave_lds_sync(); }
    };
    // (positive; the floor keeps masked scores at -inf instead of NaN should a head's K scale be zero)
    auto score_scale_of = [&](const TileUni& uc) __attribute__((always_inline)) {
        return fmaxf(a.sm_scale_log2 * ((KV8 && k_scale) ? k_scale[uc.kvr] : 1.0f), 1e-30f);
    };
    // ================= first tile of a piece =================
    auto open_piece = [&](const TileUni& uc) __attribute__((always_inline)) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) { qhi[ks] = n < G ? qnext[ks] : make_uint4(0, 0, 0, 0); qlo[ks] = make_uint4(0, 0, 0, 0); }
        if (ROPE_Q) {
            float sn1, cs1;
            sincosf((float)(uc.seq_len - 1 + a.step_mode) * lane_freq, &sn1, &cs1); // q sits at the last token
            wave_lds_sync(); // the previous piece's reads of the table are done
            rope_cs[0][lane] = cs1;
            rope_cs[ROPE_Q ? 1 : 0][lane] = sn1; // (the index keeps the one-row dummy of the other instantiations in bounds)
            wave_lds_sync();
        }
        if (ROPE_Q && n < G) {
            // the rotated q is split into a storage-precision head and tail (q = hi + lo) and both are
            // contracted, so rotating inside the kernel costs no precision
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) { // dims d = 32ks+8j+e pair with d+64, held at ks+2
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    float x[2] = {M::unpack_lo(u4(qhi[ks], w)), M::unpack_hi(u4(qhi[ks], w))};
                    float y[2] = {M::unpack_lo(u4(qhi[ks + 2], w)), M::unpack_hi(u4(qhi[ks + 2], w))};
                    float xr[2], yr[2];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const float c = rope_cs[0][d_of(ks) + 2 * w + e], s = rope_cs[ROPE_Q ? 1 : 0][d_of(ks) + 2 * w + e];
                        rope_pair(x[e], y[e], c, s, xr[e], yr[e]);
                    }
                    const uint32_t xh = M::pack2(xr[0], xr[1]), yh = M::pack2(yr[0], yr[1]);
                    u4(qhi[ks], w) = xh;
                    u4(qhi[ks + 2], w) = yh;
                    u4(qlo[ks], w) = M::pack2(xr[0] - M::unpack_lo(xh), xr[1] - M::unpack_hi(xh));
                    u4(qlo[ks + 2], w) = M::pack2(yr[0] - M::unpack_lo(yh), yr[1] - M::unpack_hi(yh));
                }
            }
        }
        m_run = -INFINITY;
        l_run = 0.f;
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    };
    // ---- scores: S^T[token][head], lane (head n, group j) gets tokens 16u + 4j + r
    auto scores = [&](const uint4 (&kop)[2][4], f32x4_t (&s)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            s[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) s[u] = M::run(kop[u][ks], qhi[ks], s[u]);
            if (ROPE_Q) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) s[u] = M::run(kop[u][ks], qlo[ks], s[u]);
            }
        }
    };
    // Rows of finished pieces leave in one go at the end of the slot.  A store in the middle of the stream is
    // expensive out of proportion on this target: loads and stores share one in-order counter, so the data of
    // every load issued after a store is held back until the store has been acknowledged, and under a full read
    // stream that takes longer than a tile -- measured 2.3 us per piece, wherever in the tile loop the stores
    // were placed, non-temporal or not.
    int pend_rows = 0, pend_n = 0;
    // rows [row0, row0 + rows) of the parked rows to dst, their log-sum-exps to lse_p (all arguments wave-uniform)
    auto store_piece = [&](char* dst_c, float* lse_p, int row0, int rows, bool f32) __attribute__((always_inline)) {
        const float* src = stage_lds + row0 * kStageRow;
        if (f32) { // fp32 rows, four elements per lane; the rows lie side by side at the destination
            float* dst = reinterpret_cast<float*>(dst_c);
            for (int c = lane; c < rows * 32; c += 64) {
                const int row = c >> 5, w = c & 31;
                const float4 v = *reinterpret_cast<const float4*>(src + row * kStageRow + 4 * w);
                store_global_16(dst + row * 128 + 4 * w, v.x, v.y, v.z, v.w);
            }
        } else if constexpr (!std::is_same<OT, float>::value) { // 16-bit rows, eight elements per lane
            OT* dst = reinterpret_cast<OT*>(dst_c);
            for (int c = lane; c < rows * 16; c += 64) {
                const int row = c >> 4, w = c & 15;
                const float4 x = *reinterpret_cast<const float4*>(src + row * kStageRow + 8 * w);
                const float4 y = *reinterpret_cast<const float4*>(src + row * kStageRow + 8 * w + 4);
                uint4 o;
                o.x = (uint32_t)StoreCvt<OT>::from(x.x).bits | ((uint32_t)StoreCvt<OT>::from(x.y).bits << 16);
                o.y = (uint32_t)StoreCvt<OT>::from(x.z).bits | ((uint32_t)StoreCvt<OT>::from(x.w).bits << 16);
                o.z = (uint32_t)StoreCvt<OT>::from(y.x).bits | ((uint32_t)StoreCvt<OT>::from(y.y).bits << 16);
                o.w = (uint32_t)StoreCvt<OT>::from(y.z).bits | ((uint32_t)StoreCvt<OT>::from(y.w).bits << 16);
                store_global_16(dst + row * 128 + 8 * w, __uint_as_float(o.x), __uint_as_float(o.y), __uint_as_float(o.z),
                                __uint_as_float(o.w));
            }
        }
        if (lse_p && lane < rows)
            *(__attribute__((address_space(1))) float*)(lse_p + lane) = stage_lds[kStageRows * kStageRow + row0 + lane];
    };
    auto store_rows = [&]() __attribute__((always_inline)) {
        for (int pc = 0; pc < pend_n; ++pc) {
            const StagedPiece sp = stage_desc[pc]; // (the same in every lane)
            store_piece(sp.dst, sp.lse, __builtin_amdgcn_readfirstlane(sp.row0), __builtin_amdgcn_readfirstlane(sp.rows),
                        __builtin_amdgcn_readfirstlane(sp.f32) != 0);
        }
        wave_lds_sync(); // everything parked has been read before anything new is parked
        pend_rows = 0;
        pend_n = 0;
    };
    // ---- mask, online softmax, O += P V (V of the tile is in LDS), and the rows of a finished piece
    auto softmax_pv = [&](const TileUni& uc, f32x4_t (&s)[2], float score_scale, bool last_of_slot) __attribute__((always_inline)) {
        const int tile_tok0 = uc.t * kTileTok, tok_end = uc.tok_end;
        const bool ragged = tile_tok0 + kTileTok > tok_end; // wave-uniform
        if (ragged) {
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (tile_tok0 + 16 * u + 4 * j + r >= tok_end) s[u][r] = -INFINITY;
        }
        float tmax = -INFINITY; // (a running maximum compiles to v_max3 pairs; a tree of fmaxf does not)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r) tmax = fmaxf(tmax, s[u][r]);
        // the scores stay unscaled in registers: the scale is applied to the maximum here and to every
        // score inside the fused multiply-add that feeds exp2
        tmax = lane_max_xor32(lane_max_xor16(tmax)) * score_scale;
        // finite also for a tile without live tokens (one past the present end under a table that runs
        // ahead): its probabilities and alpha come out 0 instead of NaN
        const float m_new = fmaxf(fmaxf(m_run, tmax), -1e30f);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new); // 0 on the first tile (m_run = -inf)
        // The probabilities enter the second contraction as a storage-precision head plus tail
        // (p = hi + lo, two MFMAs per block): the matrix cores cost nothing here and the result
        // keeps fp32-level accuracy instead of the 8 to 11 bits of a single rounded operand.
        float psum = 0.f;
        uint4 pa, pb;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(s[u][0], score_scale, -m_new));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(s[u][1], score_scale, -m_new));
            const float p2 = __builtin_amdgcn_exp2f(fmaf(s[u][2], score_scale, -m_new));
            const float p3 = __builtin_amdgcn_exp2f(fmaf(s[u][3], score_scale, -m_new));
            psum += (p0 + p1) + (p2 + p3);
            const uint32_t h01 = M::pack2(p0, p1), h23 = M::pack2(p2, p3);
            u4(pa, 2 * u) = h01;
            u4(pa, 2 * u + 1) = h23;
            u4(pb, 2 * u) = M::pack2(p0 - M::unpack_lo(h01), p1 - M::unpack_hi(h01));
            u4(pb, 2 * u + 1) = M::pack2(p2 - M::unpack_lo(h23), p3 - M::unpack_hi(h23));
        }
        psum = lane_sum_xor32(lane_sum_xor16(psum));
        l_run = l_run * alpha + psum;
        m_run = m_new;

        // ---- rescale the output rows (head 4j+i lives in lane 4j+i of the score layout)
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float al = __shfl(alpha, 4 * j + i, 64);
#pragma unroll
                for (int d = 0; d < 8; ++d) acc[d][i] *= al;
            }
        }
        wave_lds_sync(); // V tile written before the transposed reads
        // ---- O[head][d] += P[head][tok] V[tok][d], eight 16-wide d blocks
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            uint4 vb;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const unsigned char* src = v_lds + (16 * u + 4 * j + (n >> 2)) * kVRowBytes + d * 32 + (n & 3) * 8;
                const s16x4_t tr = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (s16x4_t __attribute__((address_space(3)))*)(src));
                const uint2 w = __builtin_bit_cast(uint2, tr);
                u4(vb, 2 * u) = w.x;
                u4(vb, 2 * u + 1) = w.y;
            }
            acc[d] = M::run(pa, vb, acc[d]);
            acc[d] = M::run(pb, vb, acc[d]);
        }

        if (uc.flags & 2) { // ================= last tile of a piece: final rows, or the split-K partial
            const int b = uc.seq, kvh = uc.kvh, partial = uc.partial;
            const float inv_l = (l_run > 0.f ? 1.0f / l_run : 0.f) * ((KV8 && v_scale) ? v_scale[uc.kvr] : 1.0f);
            const float lse2 = l_run > 0.f ? m_run + log2f(l_run) : -INFINITY;
            // the normalised rows are parked in LDS, head-major (store_rows above says why)
            if (pend_rows + G > kStageRows || pend_n == kStagePieces) store_rows();
            float* rows = stage_lds + pend_rows * kStageRow;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int head = 4 * j + i;
                const float il = __shfl(inv_l, head, 64);
                if (head < G) {
#pragma unroll
                    for (int d = 0; d < 8; ++d) rows[head * kStageRow + d * 16 + n] = acc[d][i] * il;
                }
            }
            if (j == 0 && n < G) stage_lds[kStageRows * kStageRow + pend_rows + n] = partial < 0 ? lse2 * 0.6931471805599453f : lse2;
            const bool f32_rows = partial >= 0 || std::is_same<OT, float>::value;
            char* dst_c;
            float* lse_p;
            if (partial >= 0) {
                dst_c = reinterpret_cast<char*>(a.part_o + (size_t)partial * 16 * 128);
                lse_p = a.part_lse + (size_t)partial * 16;
            } else {
                dst_c = reinterpret_cast<char*>(reinterpret_cast<OT*>(a.out) + ((size_t)b * a.num_qo_heads + kvh * G) * 128);
                lse_p = a.lse ? a.lse + (size_t)b * a.num_qo_heads + kvh * G : nullptr;
            }
            if (last_of_slot) { // nothing comes after these stores: out they go, behind whatever is still parked
                wave_lds_sync();
                const int row0 = pend_rows;
                if (pend_n) store_rows();
                store_piece(dst_c, lse_p, row0, G, f32_rows);
            } else {
                if (lane == 0) {
                    StagedPiece sp;
                    sp.dst = dst_c; sp.lse = lse_p;
                    sp.row0 = pend_rows; sp.rows = G; sp.f32 = f32_rows ? 1 : 0; sp.pad = 0;
                    stage_desc[pend_n] = sp;
                }
                wave_lds_sync();
                pend_rows += G;
                ++pend_n;
            }
        }
    };

    if constexpr (KV8) {
        // ---- one-byte pools: two tiles in flight.  Tile g lives in set (g - g_begin) % 2; its set is refilled with
        // tile g + 2 as soon as its bytes have been widened into operand registers (K) and parked in LDS (V).
        TileUni dA = un, dB = un; // descriptions of the tiles in sets 0 and 1
        {
            const bool second = g_begin + 1 < g_end;
            if (second) dB = read_info(0, 1);
            issue_loads_kv8(tile_base(dB), std::integral_constant<int, 1>{}, second);
        }
        auto body = [&](int g, auto set_c, auto last_c) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_c)::value;
            constexpr bool LAST = decltype(last_c)::value; // the copy behind the loop: nothing left to fetch
            const TileUni uc = SET ? dB : dA;
            const int i = g - chunk_base;
            // the tile after next, which takes over this set
            const bool more = !LAST && g + 2 < g_end;
            TileUni u2 = uc;
            if (more) u2 = read_info(i + 2 >= kInfoChunk ? buf ^ 1 : buf, (i + 2) & (kInfoChunk - 1));
            const TileBase nb = tile_base(u2);
            __builtin_amdgcn_sched_barrier(0);
            if (!LAST) info_traffic(i);
            const float score_scale = score_scale_of(uc);
            if (uc.flags & 1) open_piece(uc);

            const int tile_tok0 = uc.t * kTileTok;
            const bool ragged = tile_tok0 + kTileTok > uc.tok_end; // wave-uniform
            wave_lds_sync(); // transposed reads of the previous tile come before V is overwritten
            if (!ragged) {
#pragma unroll
                for (int w = 0; w < 4; ++w) { // 16 e4m3 bytes -> 16 operand-type values -> 32 B of the LDS row
                    unsigned char* dst = v_lds + (8 * w + (lane >> 3)) * kVRowBytes + (lane & 7) * 32;
                    *reinterpret_cast<uint4*>(dst) = fp8x8_to_op<BF16>(vreg[4 * SET + w], 0);
                    *reinterpret_cast<uint4*>(dst + 16) = fp8x8_to_op<BF16>(vreg[4 * SET + w], 1);
                }
            } else {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    uint4 v = vreg[4 * SET + w];
                    const int row = 8 * w + (lane >> 3);
                    if (tile_tok0 + row >= uc.tok_end) v = make_uint4(0, 0, 0, 0); // 0 * garbage must be 0
                    unsigned char* dst = v_lds + row * kVRowBytes + (lane & 7) * 32;
                    *reinterpret_cast<uint4*>(dst) = fp8x8_to_op<BF16>(v, 0);
                    *reinterpret_cast<uint4*>(dst + 16) = fp8x8_to_op<BF16>(v, 1);
                }
            }
            uint4 kcur[2][4];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) kcur[u][ks] = fp8x8_to_op<BF16>(kreg[u][2 * SET + (ks >> 1)], ks & 1);
            // the set is free: q rows of the next tile's piece (one tile ahead), K/V of the tile after next
            if constexpr (!LAST) {
                if (g + 1 < g_end) {
                    const TileUni& u1 = SET ? dA : dB;
                    if (u1.flags & 1) issue_q(u1);
                }
                issue_loads_kv8(nb, set_c, more);
                if (SET) dB = u2; else dA = u2;
                if (i + 1 == kInfoChunk) { chunk_base += kInfoChunk; buf ^= 1; }
            }
            f32x4_t s[2];
            scores(kcur, s);
            softmax_pv(uc, s, score_scale, g + 1 == g_end);
        };
        // (The loop has no exit between its halves, so that the only way into one set's half is through the
        // other set's half: the waits the compiler places for a set's registers then leave the other set's loads
        // in flight.  An odd last tile gets a copy of the body of its own.)
        int g = g_begin;
        for (; g + 1 < g_end; g += 2) {
            body(g, std::integral_constant<int, 0>{}, std::false_type{});
            body(g + 1, std::integral_constant<int, 1>{}, std::false_type{});
        }
        if (g < g_end) body(g, std::integral_constant<int, 0>{}, std::true_type{});
    } else {
        for (int g = g_begin; g < g_end; ++g) {
            const TileUni uc = un; // the tile computed in this iteration (its loads are in flight or done)
            const int i = g - chunk_base;
            // The description and the addresses of the next tile come first, while this tile's data is
            // still on its way: the time between its arrival and the next loads is time in which this
            // wave has nothing in flight.
            TileBase nb;
            if (g + 1 < g_end) {
                const int nbuf = (i + 1 == kInfoChunk) ? buf ^ 1 : buf;
                un = read_info(nbuf, (i + 1) & (kInfoChunk - 1));
                nb = tile_base(un);
            }
            __builtin_amdgcn_sched_barrier(0);
            info_traffic(i);
            const float score_scale = score_scale_of(uc);
            if (uc.flags & 1) open_piece(uc);

            // ================= one tile =================
            const int tile_tok0 = uc.t * kTileTok;
            const bool ragged = tile_tok0 + kTileTok > uc.tok_end; // wave-uniform
            wave_lds_sync(); // transposed reads of the previous tile come before V is overwritten
            // (the masked variant sits behind a wave-uniform branch: written as one predicated sequence it costs
            // eight register moves and an exec-mask round trip per row on every tile, between the arrival of a
            // tile and the next loads)
            if (!ragged) {
#pragma unroll
                for (int w = 0; w < 8; ++w)
                    *reinterpret_cast<uint4*>(v_lds + (4 * w + j) * kVRowBytes + n * 16) = vreg[w];
            } else {
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    uint4 v = vreg[w];
                    if (tile_tok0 + 4 * w + j >= uc.tok_end) v = make_uint4(0, 0, 0, 0); // 0 * garbage must be 0
                    *reinterpret_cast<uint4*>(v_lds + (4 * w + j) * kVRowBytes + n * 16) = v;
                }
            }
            // The K rows are contracted straight out of their landing registers and the next tile's loads go
            // out right behind the eight score instructions (which have read their operands by then).
            // Every load of this wave has arrived by now (the V rows just parked were the youngest).  Said
            // explicitly, because the compiler's bookkeeping merges paths on which it cannot tell: without this
            // it guards the landing registers it reuses as address temporaries further down with waits that
            // count loads from the wrong end -- no-ops on most tiles, but where a new piece's q rows have just
            // been requested they held the next tile's V loads back until q had arrived.
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0)
            f32x4_t s[2];
            scores(kreg, s);
            __builtin_amdgcn_sched_barrier(0); // the loads below overwrite the operands of the instructions above
            if (g + 1 < g_end) {
                if (i + 1 == kInfoChunk) { chunk_base += kInfoChunk; buf ^= 1; }
                if (un.flags & 1) issue_q(un); // next tile opens a new piece
                issue_loads(nb);
            }
            softmax_pv(uc, s, score_scale, g + 1 == g_end);
        }
    }
    store_rows(); // every piece the slot has finished since the last time
}

// Combine the partials of one split (sequence, kv head): o = sum_i o_i 2^(lse_i - M) / sum_i 2^(lse_i - M).
// One workgroup per (split, q head of the group): 128 lanes (one per output dimension) x S slices.  A
// slice fetches eight partials at a time with all loads issued before any is used and merges them with a
// running maximum; slice s takes batches s, s+S, ...  With S = 1 (splits of up to 16 partials, what large
// batches produce) that is two dependent memory round trips for up to eight partials.  A single long
// sequence at small batch is cut into as many pieces as there are wave slots (256 partials per kv head
// for one sequence on the whole chip): S = 4 or 8 slices then work side by side and are merged through
// LDS, instead of 32 round trips one after the other.  (Batches of 32 per lane were measured as well:
// slower on the large-batch workload, where most splits have two to four partials.)
template <typename OT, int S>
__global__ __launch_bounds__(128 * S) void decode_mfma_combine_kernel(const MfmaCombine* __restrict__ combos,
                                                                      const float* __restrict__ part_o,
                                                                      const float* __restrict__ part_lse, void* out,
                                                                      float* lse, uint32_t num_qo_heads, uint32_t G) {
    const MfmaCombine c = combos[blockIdx.x];
    const uint32_t g = blockIdx.y, d = threadIdx.x, sl = threadIdx.y;
    float M = -INFINITY, wsum = 0.f, o = 0.f;
    for (int i0 = 8 * (int)sl; i0 < c.count; i0 += 8 * S) {
        float li[8], oi[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const bool live = i0 + k < c.count;
            const size_t slot = (size_t)(c.first + (live ? i0 + k : 0));
            li[k] = live ? part_lse[slot * 16 + g] : -INFINITY;
            oi[k] = live ? part_o[(slot * 16 + g) * 128 + d] : 0.f;
        }
        float m2 = M;
#pragma unroll
        for (int k = 0; k < 8; ++k) m2 = fmaxf(m2, li[k]);
        if (m2 == -INFINITY) continue;
        const float sc = exp2f(M - m2); // 0 while nothing has been merged yet
        wsum *= sc;
        o *= sc;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float w = exp2f(li[k] - m2); // -inf -> 0
            wsum += w;
            o += w * oi[k];
        }
        M = m2;
    }
    if constexpr (S > 1) {
        __shared__ float sm_m[S][128], sm_w[S][128], sm_o[S][128];
        sm_m[sl][d] = M;
        sm_w[sl][d] = wsum;
        sm_o[sl][d] = o;
        __syncthreads();
        if (sl != 0) return;
        float mm = -INFINITY;
#pragma unroll
        for (int t = 0; t < S; ++t) mm = fmaxf(mm, sm_m[t][d]);
        wsum = 0.f;
        o = 0.f;
        if (mm != -INFINITY) {
#pragma unroll
            for (int t = 0; t < S; ++t) {
                const float sc = exp2f(sm_m[t][d] - mm); // an empty slice has M = -inf: weight 0
                wsum += sm_w[t][d] * sc;
                o += sm_o[t][d] * sc;
            }
        }
        M = mm;
    }
    o = wsum > 0.f ? o / wsum : 0.f;
    const size_t hq = (size_t)c.seq * num_qo_heads + (size_t)c.kvh * G + g;
    reinterpret_cast<OT*>(out)[hq * 128 + d] = StoreCvt<OT>::from(o);
    if (lse && d == 0) lse[hq] = (M + log2f(wsum)) * 0.6931471805599453f;
}

// ---- second half of the one-call decode step -------------------------------------------------------------
// The decode kernel above has attended over every token but the newest of each sequence and left one partial
// result per piece.  This kernel takes the newest token from the caller's rows instead of from the pool: it
// rotates the new K row (and q, in registers) at position seq_len-1, writes K and V into their page slot -- the
// append -- and folds the token's own term exp(q.k) v into the merge of the partials.  One workgroup per
// (sequence, scheduled unit, group of HB q heads): 32 lanes per head with four output dimensions each, x S slices
// over the partials (thread layout below).  The appended rows carry the same bits the append kernel writes.
template <typename T> __device__ __forceinline__ float pool_to_f32(T v) { return to_f32(v); }
template <> __device__ __forceinline__ float pool_to_f32<e4m3_t>(e4m3_t v) {
    return __builtin_amdgcn_cvt_f32_fp8((int)v.bits, 0);
}
template <typename T> __device__ __forceinline__ T pool_from_f32(float f) { return StoreCvt<T>::from(f); }
template <> __device__ __forceinline__ e4m3_t pool_from_f32<e4m3_t>(float f) { return e4m3_t{f32_to_e4m3_bits(f)}; }

struct StepFinishArgs {
    const void* q;
    const void* k_new;
    const void* v_new;
    char* k_data;
    char* v_data;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    const int32_t* steps_ahead;
    const MfmaUnit* units;
    const float* part_o;   // [pieces][16][128]
    const float* part_lse; // [pieces][16]
    void* out;
    float* lse;
    const float* k_scale;
    const float* v_scale;
    uint64_t stride_page, stride_n, stride_h;
    uint32_t page_size, num_qo_heads, num_kv_heads, group, parts;
    int rope;
    float sm_scale_log2;
    alignas(8) RopeFreqs freqs; // (read two at a time)
};

// Thread layout: 32 lanes per q head, four consecutive output dimensions per lane (16-byte loads of the partial
// rows); HB heads of the unit share a workgroup (threadIdx.y) and with it the angles of the new token's
// position; S slices (threadIdx.z) split a long list of partials.  The kernel is short enough that the number
// of instructions its waves issue, not the bytes they move, sets its duration.
template <typename T> __device__ __forceinline__ void load4_f32(const T* p, float* f) { // four 16-bit elements
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    f[0] = to_f32(T{(uint16_t)(w.x & 0xffffu)});
    f[1] = to_f32(T{(uint16_t)(w.x >> 16)});
    f[2] = to_f32(T{(uint16_t)(w.y & 0xffffu)});
    f[3] = to_f32(T{(uint16_t)(w.y >> 16)});
}
template <typename T> __device__ __forceinline__ void store4(T* p, const T* v) { // four 16-bit elements
    *reinterpret_cast<uint2*>(p) = make_uint2((uint32_t)v[0].bits | ((uint32_t)v[1].bits << 16),
                                              (uint32_t)v[2].bits | ((uint32_t)v[3].bits << 16));
}
template <> __device__ __forceinline__ void store4<e4m3_t>(e4m3_t* p, const e4m3_t* v) {
    *reinterpret_cast<uint32_t*>(p) = (uint32_t)v[0].bits | ((uint32_t)v[1].bits << 8) | ((uint32_t)v[2].bits << 16) |
                                      ((uint32_t)v[3].bits << 24);
}
template <> __device__ __forceinline__ void store4<float>(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

template <typename QT, typename PT, typename OT, int S, int HB>
__global__ __launch_bounds__(32 * HB * S) void decode_step_finish_kernel(const MfmaUnit* __restrict__ units_p,
                                                                         const int32_t* __restrict__ ahead_p, StepFinishArgs a) {
    const uint32_t t = threadIdx.x, hl = threadIdx.y, sl = threadIdx.z;
    // The two pointers in front of the argument block arrive in registers with the wave (kernel-argument preload of
    // this target; the build asks for it), so the unit record and the step counter are asked for at once, while the
    // rest of the arguments is still being fetched.  Those, left to the compiler, are fetched a few at a time, each
    // where it is first needed and each with a wait of its own: scalar round trips in a row before the first row is
    // asked for.  The empty asm below needs a value made of all of them, so they are all asked for here, in one batch.
    const MfmaUnit u = units_p[blockIdx.x];
    // (without a step counter the record's own padding, which is zero, is read in its place: a load under a condition
    // would be waited for on the spot, before the arguments below are asked for)
    const int ahead_raw = *(ahead_p ? ahead_p : &units_p[blockIdx.x].pad[0]);
    asm volatile("" ::"s"(a.q), "s"(a.k_new), "s"(a.v_new), "s"(a.k_data), "s"(a.v_data), "s"(a.indices), "s"(a.part_o),
                 "s"(a.part_lse), "s"(a.out), "s"(a.lse), "s"(a.k_scale), "s"(a.v_scale), "s"(a.stride_page),
                 "s"(a.stride_n), "s"(a.stride_h), "s"(a.page_size), "s"(a.num_qo_heads), "s"(a.num_kv_heads),
                 "s"(a.group), "s"(a.parts), "s"(a.rope), "s"(a.sm_scale_log2));
    // The angles of the new token's position: lane t of a head works out pairs 2t and 2t + 1, and the lanes of the
    // head then pass them round (no LDS table, no workgroup barrier).  The two frequencies are asked for here, beside
    // the unit record, not where they are used.
    float2 freq2 = *reinterpret_cast<const float2*>(&a.freqs.f[2 * t]);
    const uint32_t g_raw = blockIdx.y * HB + hl;
    const bool head_live = g_raw < a.group;           // a group that is no multiple of HB leaves lanes idle
    const uint32_t g = head_live ? g_raw : a.group - 1;
    const int b = u.seq;
    const int kvr = u.unit / (int)a.parts; // the kv head whose K/V the unit reads
    const uint32_t hq = (uint32_t)u.unit * a.group + g;
    const uint32_t d0 = 4 * t;             // this lane's four output dimensions
    const bool upper = d0 >= 64;           // they are the second elements of their rotate-half pairs
    const uint32_t i0 = d0 & 63, dp = upper ? d0 - 64 : d0 + 64;
    // Everything that depends on the unit record alone is requested at once: the caller's rows, the scales
    // and the first four partial results of this slice.  (The sequence's length and its place in the page
    // list come with the unit record, from the host table the plan was made from, like the lengths the
    // decode kernel works with.)
    const int seq_len = u.seq_len - max(ahead_raw, 0);
    // (the page of the newest token is asked for beside the rows, not where it is used: one dependent round trip less
    // between the unit record and the append -- and by every workgroup, needed or not: a unit's sequence has pages,
    // and a load under a condition would be waited for on the spot)
    const bool appends = g_raw == 0 && sl == 0 && u.unit % (int)a.parts == 0; // one head's lanes per (sequence, kv head)
    const int64_t page = a.indices[u.ip0 + max(seq_len - 1, 0) / (int)a.page_size];
    const QT* qrow = reinterpret_cast<const QT*>(a.q) + ((size_t)b * a.num_qo_heads + hq) * 128;
    const QT* krow = reinterpret_cast<const QT*>(a.k_new) + ((size_t)b * a.num_kv_heads + kvr) * 128;
    const QT* vrow = reinterpret_cast<const QT*>(a.v_new) + ((size_t)b * a.num_kv_heads + kvr) * 128;
    float q_own[4], q_par[4], k_own[4], k_par[4], v_in[4];
    load4_f32(qrow + d0, q_own);
    load4_f32(qrow + dp, q_par);
    load4_f32(krow + d0, k_own);
    load4_f32(krow + dp, k_par);
    load4_f32(vrow + d0, v_in);
    const float ksc = a.k_scale ? a.k_scale[kvr] : 1.0f, vsc = a.v_scale ? a.v_scale[kvr] : 1.0f;
    constexpr int NB = 4; // partials per batch of loads
    auto load_batch = [&](int j0, float* li, float4* oi) {
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            const bool live = j0 + k < u.count;
            const size_t slot = (size_t)(u.first_piece + (live ? j0 + k : 0));
            li[k] = live ? a.part_lse[slot * 16 + g] : -INFINITY;
            oi[k] = *reinterpret_cast<const float4*>(a.part_o + (slot * 16 + g) * 128 + d0);
        }
    };
    float li0[NB];
    float4 oi0[NB];
    load_batch(NB * (int)sl, li0, oi0);
    asm("" : "+v"(freq2.x), "+v"(freq2.y)); // (asked for at the top, kept in their registers: not fetched again where used)

    OT* orow = reinterpret_cast<OT*>(a.out) + ((size_t)b * a.num_qo_heads + hq) * 128;
    if (seq_len <= 0) { // no token at present: nothing to append, a zero row
        const OT z[4] = {StoreCvt<OT>::from(0.f), StoreCvt<OT>::from(0.f), StoreCvt<OT>::from(0.f), StoreCvt<OT>::from(0.f)};
        if (sl == 0 && head_live) store4(orow + d0, z);
        if (a.lse && sl == 0 && head_live && t == 0) a.lse[(size_t)b * a.num_qo_heads + hq] = -INFINITY;
        return;
    }
    const int pos = seq_len - 1;

    // ---- the newest token: rotated q and K elements of this lane, the bits the cache gets, the score
    float v_term[4], s_new;
    {
        float qd[4], kd[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) { qd[e] = q_own[e]; kd[e] = k_own[e]; }
        if (a.rope) {
            float sn2[2], cs2[2];
            sincosf((float)pos * freq2.x, &sn2[0], &cs2[0]);
            sincosf((float)pos * freq2.y, &sn2[1], &cs2[1]);
            const int src = (int)(i0 >> 1); // the lane of this head that holds pairs i0 and i0 + 1; the next one i0 + 2, i0 + 3
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float sn = __shfl(sn2[e & 1], src + (e >> 1), 32), cs = __shfl(cs2[e & 1], src + (e >> 1), 32);
                float xr, yr;
                rope_pair(upper ? q_par[e] : q_own[e], upper ? q_own[e] : q_par[e], cs, sn, xr, yr);
                qd[e] = upper ? yr : xr;
                rope_pair(upper ? k_par[e] : k_own[e], upper ? k_own[e] : k_par[e], cs, sn, xr, yr);
                kd[e] = upper ? yr : xr;
            }
        }
        PT k_st[4], v_st[4];
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            k_st[e] = pool_from_f32<PT>(a.k_scale ? kd[e] / ksc : kd[e]);
            v_st[e] = pool_from_f32<PT>(a.v_scale ? v_in[e] / vsc : v_in[e]);
            // the score against the K bits as cached, exactly as a later step will see them
            dot += qd[e] * pool_to_f32(k_st[e]);
            v_term[e] = pool_to_f32(v_st[e]) * vsc;
        }
        if (appends) { // the append
            const size_t off = (size_t)page * a.stride_page + (size_t)(pos % (int)a.page_size) * a.stride_n +
                               (size_t)kvr * a.stride_h + d0;
            store4(reinterpret_cast<PT*>(a.k_data) + off, k_st);
            store4(reinterpret_cast<PT*>(a.v_data) + off, v_st);
        }
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64); // over the 32 lanes of the head
        s_new = dot * a.sm_scale_log2 * ksc;
    }

    // ---- the partial results of the older tokens (normalised rows and base-2 log-sum-exp per piece)
    float M = -INFINITY, wsum = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
    auto merge_batch = [&](const float* li, const float4* oi) {
        float m2 = M;
#pragma unroll
        for (int k = 0; k < NB; ++k) m2 = fmaxf(m2, li[k]);
        if (m2 == -INFINITY) return;
        const float sc = __builtin_amdgcn_exp2f(M - m2); // 0 while nothing has been merged yet
        wsum *= sc;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] *= sc;
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            const float w = __builtin_amdgcn_exp2f(li[k] - m2); // -inf -> 0 (and the row read for a dead slot is finite)
            wsum += w;
            o[0] += w * oi[k].x;
            o[1] += w * oi[k].y;
            o[2] += w * oi[k].z;
            o[3] += w * oi[k].w;
        }
        M = m2;
    };
    merge_batch(li0, oi0);
    for (int j0 = NB * (int)sl + NB * S; j0 < u.count; j0 += NB * S) {
        float li[NB];
        float4 oi[NB];
        load_batch(j0, li, oi);
        merge_batch(li, oi);
    }
    if constexpr (S > 1) {
        __shared__ float sm_m[S][HB][32], sm_w[S][HB][32];
        __shared__ float4 sm_o[S][HB][32];
        sm_m[sl][hl][t] = M;
        sm_w[sl][hl][t] = wsum;
        sm_o[sl][hl][t] = make_float4(o[0], o[1], o[2], o[3]);
        __syncthreads();
        if (sl != 0) return;
        float mm = -INFINITY;
#pragma unroll
        for (int z = 0; z < S; ++z) mm = fmaxf(mm, sm_m[z][hl][t]);
        wsum = 0.f;
        o[0] = o[1] = o[2] = o[3] = 0.f;
        if (mm != -INFINITY) {
#pragma unroll
            for (int z = 0; z < S; ++z) {
                const float sc = __builtin_amdgcn_exp2f(sm_m[z][hl][t] - mm); // an empty slice has M = -inf: weight 0
                const float4 oz = sm_o[z][hl][t];
                wsum += sm_w[z][hl][t] * sc;
                o[0] += oz.x * sc;
                o[1] += oz.y * sc;
                o[2] += oz.z * sc;
                o[3] += oz.w * sc;
            }
        }
        M = mm;
    }
    // ---- the newest token joins with weight 2^(s_new - max)
    const float m_all = fmaxf(M, s_new);
    const float sc_old = __builtin_amdgcn_exp2f(M - m_all); // 0 when there are no older tokens
    const float w_new = __builtin_amdgcn_exp2f(s_new - m_all);
    const float denom = wsum * sc_old + w_new, inv = 1.0f / denom;
    OT res[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) res[e] = StoreCvt<OT>::from((o[e] * sc_old + w_new * v_term[e]) * inv);
    if (head_live) store4(orow + d0, res);
    if (a.lse && head_live && t == 0) a.lse[(size_t)b * a.num_qo_heads + hq] = (m_all + log2f(denom)) * 0.6931471805599453f;
}

struct DecodeArgs; // general-kernel argument block (bz_decode.hip); only its scalar fields are forwarded here

template <bool BF16, typename OT, bool ROPE_Q, bool KV8>
static void launch_mfma_k(const DecodePlan* p, const MfmaDecodeArgs& a, hipStream_t s) {
    if (p->mfma_streaming)
        hipLaunchKernelGGL((decode_mfma_kernel<BF16, OT, ROPE_Q, KV8, true>), dim3(p->mfma_slots), dim3(64), 0, s, a.heads, a,
                           (const char*)a.q, a.k_data, a.v_data, a.indices, a.pieces, a.tiles, a.k_scale,
                           a.v_scale);
    else
        hipLaunchKernelGGL((decode_mfma_kernel<BF16, OT, ROPE_Q, KV8, false>), dim3(p->mfma_slots), dim3(64), 0, s, a.heads, a,
                           (const char*)a.q, a.k_data, a.v_data, a.indices, a.pieces, a.tiles, a.k_scale,
                           a.v_scale);
}

template <bool BF16, typename OT>
static int launch_mfma(const DecodePlan* p, const MfmaDecodeArgs& a, bool kv8, hipStream_t s) {
    if (p->time_start) BZ_CHECK_HIP(hipEventRecord(p->time_start, s));
    if (kv8) {
        if (a.rope_q) launch_mfma_k<BF16, OT, true, true>(p, a, s);
        else launch_mfma_k<BF16, OT, false, true>(p, a, s);
    } else {
        if (a.rope_q) launch_mfma_k<BF16, OT, true, false>(p, a, s);
        else launch_mfma_k<BF16, OT, false, false>(p, a, s);
    }
    BZ_LAUNCH_CHECK();
    if (p->time_stop) BZ_CHECK_HIP(hipEventRecord(p->time_stop, s));
    if (a.step_mode) return 0; // the finishing kernel of the one-call step folds the partials
    if (p->mfma_combos > 0) {
        const dim3 cgrid(p->mfma_combos, a.group);
        if (p->mfma_max_count <= 16)
            hipLaunchKernelGGL((decode_mfma_combine_kernel<OT, 1>), cgrid, dim3(128, 1), 0, s, p->mfma_combos_d,
                               a.part_o, a.part_lse, a.out, a.lse, a.num_qo_heads, a.group);
        else if (p->mfma_max_count <= 64)
            hipLaunchKernelGGL((decode_mfma_combine_kernel<OT, 4>), cgrid, dim3(128, 4), 0, s, p->mfma_combos_d,
                               a.part_o, a.part_lse, a.out, a.lse, a.num_qo_heads, a.group);
        else
            hipLaunchKernelGGL((decode_mfma_combine_kernel<OT, 8>), cgrid, dim3(128, 8), 0, s, p->mfma_combos_d,
                               a.part_o, a.part_lse, a.out, a.lse, a.num_qo_heads, a.group);
        BZ_LAUNCH_CHECK();
    }
    return 0;
}

int decode_fast_path(const DecodePlan* p, const void* q, void* out, float* lse, int q_dtype, int out_dtype,
                     int rope_mode, float sm_scale_log2, const RopeFreqs& freqs, const bz_paged_kv_t* kv,
                     uint32_t num_qo_heads, const float* k_scale, const float* v_scale, float* part_o,
                     float* part_lse, bool step_mode, hipStream_t s) {
    if (!p->mfma_ok || p->mfma_slots == 0) return BZ_ERR_UNSUPPORTED;
    const bool kv8 = kv->kv_dtype == BZ_E4M3;
    if ((!kv8 && kv->kv_dtype != q_dtype) || rope_mode == BZ_ROPE_FULL) return BZ_ERR_UNSUPPORTED;
    if (!kv8 && (k_scale || v_scale)) return BZ_ERR_UNSUPPORTED;
    const uint64_t es = kv8 ? 1 : 2;
    if ((kv->stride_n * es) % 16 || (kv->stride_h * es) % 16 || (kv->stride_page * es) % 16) return BZ_ERR_UNSUPPORTED;
    if (((uintptr_t)kv->k_data | (uintptr_t)kv->v_data | (uintptr_t)q | (uintptr_t)out) % 16) return BZ_ERR_UNSUPPORTED;
    MfmaDecodeArgs a;
    a.q = q; a.out = out; a.lse = lse;
    a.k_data = (const char*)kv->k_data; a.v_data = (const char*)kv->v_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.steps_ahead = kv->steps_ahead;
    a.pieces = p->mfma_pieces_d; a.tiles = p->mfma_tiles_d; a.heads = p->mfma_heads_d;
    a.part_o = part_o; a.part_lse = part_lse; // split-K partials: the plan's float workspace or the library's own array
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.page_size = kv->page_size; a.num_qo_heads = num_qo_heads;
    a.group = num_qo_heads / kv->num_kv_heads / p->mfma_parts;
    a.rope_q = rope_mode == BZ_ROPE_Q_ONLY;
    a.step_mode = step_mode ? 1 : 0;
    a.sm_scale_log2 = sm_scale_log2;
    a.k_scale = k_scale; a.v_scale = v_scale;
    a.freqs = freqs;
    if (q_dtype == BZ_BF16)
        return out_dtype == BZ_F32 ? launch_mfma<true, float>(p, a, kv8, s) : launch_mfma<true, bf16_t>(p, a, kv8, s);
    return out_dtype == BZ_F32 ? launch_mfma<false, float>(p, a, kv8, s) : launch_mfma<false, f16_t>(p, a, kv8, s);
}

template <typename QT, typename PT, typename OT>
static int launch_step_finish(const DecodePlan* p, const StepFinishArgs& a, hipStream_t s) {
    // heads of a unit per workgroup: 4 where the group allows it (two waves), else 2 (one wave), 1 for single heads
    const uint32_t G = a.group;
    if (p->mfma_unit_max_count <= 16) { // what large batches produce
        if (G >= 4)
            hipLaunchKernelGGL((decode_step_finish_kernel<QT, PT, OT, 1, 4>), dim3(p->mfma_units, (G + 3) / 4), dim3(32, 4, 1), 0, s, a.units, a.steps_ahead, a);
        else if (G >= 2)
            hipLaunchKernelGGL((decode_step_finish_kernel<QT, PT, OT, 1, 2>), dim3(p->mfma_units, (G + 1) / 2), dim3(32, 2, 1), 0, s, a.units, a.steps_ahead, a);
        else
            hipLaunchKernelGGL((decode_step_finish_kernel<QT, PT, OT, 1, 1>), dim3(p->mfma_units, G), dim3(32, 1, 1), 0, s, a.units, a.steps_ahead, a);
    } else if (p->mfma_unit_max_count > 32 && p->mfma_unit_max_count <= 64) {
        hipLaunchKernelGGL((decode_step_finish_kernel<QT, PT, OT, 4, 2>), dim3(p->mfma_units, (G + 1) / 2), dim3(32, 2, 4), 0, s, a.units, a.steps_ahead, a);
    } else {
        // 17..32 partials (batches of eight sequences or so): eight slices, so one batch of four per slice and a single
        // round of loads, and one head per workgroup -- four waves.  Measured on 32 layers at batch 8: 497 us per step
        // against 505 with two heads per workgroup (eight waves), 527 with four (sixteen), 507 with four slices of two
        // heads.  More than 64 partials (a few very long sequences): the same shape (4 x 32 768 tokens: 90.8 against
        // 91.8 us with two heads).
        hipLaunchKernelGGL((decode_step_finish_kernel<QT, PT, OT, 8, 1>), dim3(p->mfma_units, G), dim3(32, 1, 8), 0, s, a.units, a.steps_ahead, a);
    }
    BZ_LAUNCH_CHECK();
    return 0;
}

template <typename QT, typename OT>
static int launch_step_finish_kv(const DecodePlan* p, const StepFinishArgs& a, bool kv8, hipStream_t s) {
    return kv8 ? launch_step_finish<QT, e4m3_t, OT>(p, a, s) : launch_step_finish<QT, QT, OT>(p, a, s);
}

// The one-call decode step on the matrix-core kernel: BZ_ERR_UNSUPPORTED when the shape, the plan or the
// float workspace does not allow it (the caller then runs the append and the decode as two calls).
int decode_step_fast_path(const DecodePlan* p, const void* q, const void* k_new, const void* v_new, void* out,
                          float* lse, int q_dtype, int out_dtype, int rope, float sm_scale_log2,
                          const RopeFreqs& freqs, const bz_paged_kv_t* kv, uint32_t num_qo_heads, const float* k_scale,
                          const float* v_scale, hipStream_t s) {
    if (!p->mfma_ok || p->mfma_slots == 0 || !p->mfma_units_d || p->mfma_units == 0) return BZ_ERR_UNSUPPORTED;
    // one partial per piece, in the float workspace the plan was given
    const size_t part_o_bytes = ((size_t)p->mfma_pieces * 16 * 128 * sizeof(float) + 255) / 256 * 256;
    const size_t part_lse_bytes = ((size_t)p->mfma_pieces * 16 * sizeof(float) + 255) / 256 * 256;
    if (part_o_bytes + part_lse_bytes > p->float_buffer_bytes) return BZ_ERR_UNSUPPORTED;
    float* part_o = p->mfma_part_o;
    float* part_lse = reinterpret_cast<float*>(reinterpret_cast<char*>(p->mfma_part_o) + part_o_bytes);
    const int rc = decode_fast_path(p, q, out, lse, q_dtype, out_dtype, rope ? BZ_ROPE_Q_ONLY : BZ_ROPE_NONE,
                                    sm_scale_log2, freqs, kv, num_qo_heads, k_scale, v_scale, part_o, part_lse, true, s);
    if (rc) return rc;
    StepFinishArgs a;
    a.q = q; a.k_new = k_new; a.v_new = v_new;
    a.k_data = (char*)kv->k_data; a.v_data = (char*)kv->v_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.steps_ahead = kv->steps_ahead;
    a.units = p->mfma_units_d;
    a.part_o = part_o; a.part_lse = part_lse;
    a.out = out; a.lse = lse;
    a.k_scale = k_scale; a.v_scale = v_scale;
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.page_size = kv->page_size; a.num_qo_heads = num_qo_heads; a.num_kv_heads = kv->num_kv_heads;
    a.parts = p->mfma_parts;
    a.group = num_qo_heads / kv->num_kv_heads / p->mfma_parts;
    a.rope = rope ? 1 : 0;
    a.sm_scale_log2 = sm_scale_log2;
    a.freqs = freqs;
    const bool kv8 = kv->kv_dtype == BZ_E4M3;
    if (q_dtype == BZ_BF16)
        return out_dtype == BZ_F32 ? launch_step_finish_kv<bf16_t, float>(p, a, kv8, s)
                                   : launch_step_finish_kv<bf16_t, bf16_t>(p, a, kv8, s);
    return out_dtype == BZ_F32 ? launch_step_finish_kv<f16_t, float>(p, a, kv8, s)
                               : launch_step_finish_kv<f16_t, f16_t>(p, a, kv8, s);
}

} // namespace bz
