// Ragged (causal) prefill attention on the gfx950 matrix cores: replaces
// src/kernel/attention_prefill.cu and the prefill half of flashinfer_types.cu of the BlitzScale
// worker.  head_dim 128, f16 or bf16, any number of q heads per kv head; self-attention over each request, or
// q rows for the last tokens of a request only over K/V rows for all of them (distinct ragged indices).
//
// One workgroup of 4 waves takes 128 consecutive q rows of one (request, q head); wave w owns rows
// 32w..32w+31.  K/V tiles of 32 tokens travel global -> LDS four tiles deep and are shared by the four
// waves.  Both contractions are issued "transposed" on v_mfma_f32_32x32x16:
//     S^T[kv][q] = K[kv][:] . Q[q][:]      (A = K tile from LDS,      B = Q rows from registers)
//     O^T[d][q]  = V^T[d][kv] . P^T[kv][q] (A = V tile, transposed LDS read, B = P from registers)
// so that in both results a lane's column index is its own q row: the softmax statistics, the
// rescaling of O and the P operand of the second contraction are all lane-local (the two half-waves of a
// row are joined once, at the end).
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>

#include "bz_common.hpp"

namespace bz {

typedef __attribute__((ext_vector_type(8))) __bf16 pf_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 pf_f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 pf_bf16x2;
typedef __attribute__((ext_vector_type(2))) _Float16 pf_f16x2;
typedef __attribute__((ext_vector_type(2))) float pf_f32x2;
typedef __attribute__((ext_vector_type(16))) float pf_f32x16;
typedef __attribute__((ext_vector_type(4))) short pf_s16x4;

constexpr int kBM = 128; // q rows per workgroup

// 16 bytes per lane from global memory straight into LDS: lane l's data lands at lds_addr + 16*l.
// The compiler does not know that this is a load (it would otherwise wait for every such load before
// any later LDS read, the ones of the tile in use included); the kernel waits for it explicitly.
__device__ __forceinline__ void lds_direct_load16(const char* uniform_base, uint32_t lane_offset, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_offset), "s"(uniform_base)
                 : "memory", "m0");
}

struct PrefillItem { // one workgroup's job, in launch order
    int32_t tok0;   // global index of the request's first q row
    int32_t len;    // q rows of the request (0: padding entry, nothing to do)
    int32_t q0;     // first q row of this tile, relative to the request
    int32_t head;   // q head
    int32_t kv0;    // global index of the request's first K/V row
    int32_t kv_len; // K/V rows of the request (>= len); q row i sits at position kv_len - len + i
    int32_t pad[2];
};

struct PrefillPlan {
    bool planned = false;
    bool bf16_head_tail = false; // bf16: probabilities as head + tail of bf16 instead of V widened to f16 (bz_prefill_plan_set_bf16_mode)
    uint32_t batch_size = 0, num_qo_heads = 0, num_kv_heads = 0, head_dim = 0, num_items = 0;
    uint32_t total_tokens = 0, total_kv_tokens = 0, max_len = 0; // max_len: longest K/V length
    const PrefillItem* items_d = nullptr;
    // cos / sin of position * frequency for every position a request of this batch has (float workspace), written by
    // every attention call that rotates q, on its own stream, in front of the attention kernel
    float* rope_table = nullptr; // [32 couples of pairs][max_len] x (cos, sin, cos, sin); nullptr: the float workspace has no room
    std::vector<PrefillItem> h_items; // host copy of the last job list (kept between calls)
    void* staging = nullptr;
    size_t staging_bytes = 0;
    hipEvent_t upload_done = nullptr;
    hipEvent_t time_start = nullptr, time_stop = nullptr; // optional: bracket the attention kernel's launch
};

struct PrefillArgs {
    void* out;
    const PrefillItem* items;
    const float4* rope_table; // ROPE_Q: [32 couples of pairs][rope_pitch positions] x (cos i, sin i, cos i+1, sin i+1), i even
    uint32_t rope_pitch;
    uint32_t num_qo_heads, num_kv_heads;
    int causal;
    float sm_scale_log2;
};

// Keeps a value where it is computed: the compiler would otherwise sink the packs of the first half of an
// iteration to their first use in the second and keep sixteen fp32 probabilities alive meanwhile.  (The pack
// itself stays the compiler's: written as inline assembly, v_cvt_pk_bf16_f32 returned wrong values in the first
// lanes of each half-wave -- the compiler adds wait states behind it that it cannot add behind an opaque
// instruction.)
__device__ __forceinline__ uint32_t pf_keep_here(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

template <bool BF16> struct PfMma;
template <> struct PfMma<false> {
    __device__ static __forceinline__ pf_f32x16 run(uint4 a, uint4 b, pf_f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_f16x8, a), __builtin_bit_cast(pf_f16x8, b), c,
                                                      0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        const pf_f16x2 h = __builtin_convertvector(pf_f32x2{lo, hi}, pf_f16x2);
        return __builtin_bit_cast(uint32_t, h);
    }
    __device__ static __forceinline__ uint32_t pack2_here(float lo, float hi) { return pf_keep_here(pack2(lo, hi)); }
    // acc + the two values of a packed word (v_dot2c_f32_f16 with ones: products and sum exact in fp32)
    __device__ static __forceinline__ float add_pair(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(pf_f16x2, w), pf_f16x2{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
    }
    __device__ static __forceinline__ float lo(uint32_t w) { return (float)__builtin_bit_cast(pf_f16x2, w)[0]; }
    __device__ static __forceinline__ float hi(uint32_t w) { return (float)__builtin_bit_cast(pf_f16x2, w)[1]; }
};
template <> struct PfMma<true> {
    __device__ static __forceinline__ pf_f32x16 run(uint4 a, uint4 b, pf_f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, a), __builtin_bit_cast(pf_bf16x8, b),
                                                       c, 0, 0, 0);
    }
    __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
        const pf_bf16x2 b = __builtin_convertvector(pf_f32x2{lo, hi}, pf_bf16x2); // v_cvt_pk_bf16_f32, round to nearest even
        return __builtin_bit_cast(uint32_t, b);
    }
    __device__ static __forceinline__ uint32_t pack2_here(float lo, float hi) { return pf_keep_here(pack2(lo, hi)); }
    __device__ static __forceinline__ float add_pair(uint32_t w, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(pf_bf16x2, w), pf_bf16x2{(__bf16)1.0f, (__bf16)1.0f}, acc, false);
    }
    __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};

__device__ __forceinline__ uint32_t& pf_u4(uint4& v, int i) { return reinterpret_cast<uint32_t*>(&v)[i]; }

// XOR applied to the 16-byte chunk index of V rows in LDS, by row % 4: 0, 4, 10, 14 (see the staging comment)
#define BZ_VSWZ(r) (((r) << 2) ^ (((r) >> 1) << 1))

// ---------------------------------------------------------------------------------------------------------
// The attention kernel.  A wave's instruction stream for tile j is one interleaved, software-pipelined sequence
//     8 x { matrix: S(j+1) += K(j+1) Q^T step i | LDS: next operand | vector: exp, pack, row sum of S(j) }
//     8 x { matrix: O += V(j)^T P(j)^T step i   | LDS: next operand }
// so that a wave always has matrix instructions in flight while it does its vector work: a wave issues about one
// instruction per five cycles whatever its kind, a matrix instruction keeps the pipe busy for 32, and the matrix
// and vector instructions of the two waves of a SIMD (two workgroups per CU) share one issue port, so the vector
// work has to sit in the shadow of the matrix instructions of the same wave to be free.  Operands come from LDS
// through two rings of four registers each, read four matrix instructions ahead of their use.  Tiles are copied
// global -> LDS with LDS-direct loads, kSNK (K) and kSNV (V) tiles deep, two to three tiles (about two
// microseconds) ahead of their first read; there is one workgroup barrier per tile, at the top of the iteration,
// where the tiles read next are published and the buffers of the tiles just finished are handed back to the
// copies.  The steady state (`full`) has no conditions in it; everything ragged or masked goes through `generic`.
//
// Softmax without a maximum per tile: q rows that are rotated here carry sm_scale * log2(e) in the one rounding of
// the rotated row (rows that arrive as they are keep their bits and the scale stays on the score), and the first
// score instruction of a tile accumulates onto `cinit`, a block of registers that holds -m_run, so the scores leave
// the matrix pipe as base-2 logits relative to the reference maximum m_run of their row and go into v_exp_f32 as
// they are.  m_run is set from the first tile and moved only when it has to be: a tile's probabilities are computed
// on the assumption that no score exceeds m_run by 15 or more (p < 2^15 fits the 16-bit operand of the second
// contraction and fp32 sums); the row sums, which are needed anyway, tell whether it held, and a wave for which it
// did not takes the tile's maximum, moves m_run, rescales its accumulators and computes the tile's probabilities
// again (move_maximum: rare, wave-uniform).  m_run never exceeds the true running maximum, so the largest
// probability of a row so far is always at least 1.
//
// LDS layout of a tile: 32 rows of 256 bytes, unpadded (an LDS-direct load writes 64 x 16 B to consecutive LDS);
// what keeps the operand reads free of bank conflicts is an XOR on the 16-byte column chunk:
//   K: chunk c of row r sits at position c ^ (r % 16)      (16 lanes read 16 rows, one chunk each)
//   V: chunk c of row r sits at position c ^ g(r % 4), g = 0, 4, 10, 14 (BZ_VSWZ).  The transposing read
//      ds_read_b64_tr_b16 takes 8 B per lane; a 16-lane group reads 4 rows x 32 B and two groups (4 rows x 64 B) go
//      through the 64 banks together, so the 8 (row, group) pieces must land in 8 different 32-byte bank groups
// and a lane of the copy simply fetches the chunk that belongs at its position.
constexpr int kSN = 32;                      // kv tokens per tile
constexpr int kSTile = kSN * 256;            // bytes of one K or V tile in LDS
#ifndef BZ_PF_NK
#define BZ_PF_NK 4
#endif
#ifndef BZ_PF_NV
#define BZ_PF_NV 4
#endif
constexpr int kSNK = BZ_PF_NK, kSNV = BZ_PF_NV; // K and V tiles in flight per workgroup
constexpr int kSLds = (kSNK + kSNV) * kSTile;   // 65 536 bytes per workgroup: K slots, then V slots
static_assert(kSNK == 4 && kSNV == 4, "the steady state is unrolled over four slots");

__device__ __forceinline__ void lds_direct_load16x2(const char* uniform_base, uint32_t o0, uint32_t o1, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %3\n\t"
                 "global_load_lds_dwordx4 %2, %3 offset:1024"
                 :
                 : "s"(lds_addr), "v"(o0), "v"(o1), "s"(uniform_base)
                 : "memory", "m0");
}
// Loads the compiler keeps no count of: the kernel waits for them itself (sp_wait_copies counts them like copies),
// so that a wait for the q rows does not become a wait for every tile copy in flight.  The registers must not be
// read before sp_loads_arrived() has been passed over them.
__device__ __forceinline__ uint4 sp_load16(const void* p) {
    typedef uint32_t __attribute__((ext_vector_type(4))) u32x4;
    u32x4 r;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(p) : "memory");
    return make_uint4(r.x, r.y, r.z, r.w);
}
__device__ __forceinline__ float2 sp_load8(const void* p) {
    typedef float __attribute__((ext_vector_type(2))) f32x2;
    f32x2 r;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(r) : "v"(p) : "memory");
    return make_float2(r.x, r.y);
}
__device__ __forceinline__ void sp_loads_arrived(uint4& r) { asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w)); }
__device__ __forceinline__ void sp_loads_arrived(float2& r) { asm volatile("" : "+v"(r.x), "+v"(r.y)); }

// workgroup barrier that the compiler moves no memory access across (it waits for nothing by itself)
__device__ __forceinline__ void sp_barrier() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}
// wait until at most `tiles` of this wave's tile copies (two instructions each) are still in flight
__device__ __forceinline__ void sp_wait_copies(int tiles) {
    __builtin_amdgcn_sched_barrier(0);
    switch (tiles) {
        case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
        case 1: __builtin_amdgcn_s_waitcnt(0x0F72); break;
        case 2: __builtin_amdgcn_s_waitcnt(0x0F74); break;
        case 3: __builtin_amdgcn_s_waitcnt(0x0F76); break;
        case 4: __builtin_amdgcn_s_waitcnt(0x0F78); break;
        case 5: __builtin_amdgcn_s_waitcnt(0x0F7A); break;
        case 6: __builtin_amdgcn_s_waitcnt(0x0F7C); break;
        default: __builtin_amdgcn_s_waitcnt(0x0F7E); break;
    }
    __builtin_amdgcn_sched_barrier(0);
}
// Copies are issued in pairs (K(i + kSNK), V(i + kSNV - 1)) at the top of iteration i, the first kSNK pairs
// (i = -kSNK .. -1, tiles below 0 left out) in the prologue.  The tiles first read in iteration j are K(j+2) and
// V(j); with V_NEXT also V(j+1), which is then converted in place during iteration j.  This counts the copies that
// exist (tile < n) behind the last of them, up to those of iteration j-1.
__device__ __forceinline__ int sp_copies_behind(int j, int n, bool v_next) {
    const int pk = 2 * (j + 2 - kSNK), pv = 2 * (j + 1 - kSNV) + 1; // positions of K(j+2), V(j) in the issue order
    int p = max(pk, pv);
    if (v_next && j + 1 < n) p = max(p, pv + 2);
    int c = 0;
    for (int pos = p + 1; pos <= 2 * j - 1; ++pos) {
        const int i = pos >> 1; // (arithmetic shift: positions may be negative in the first iterations)
        const int tile = (pos & 1) ? i + kSNV - 1 : i + kSNK;
        c += (tile >= 0 && tile < n) ? 1 : 0;
    }
    return c;
}
constexpr int sp_copies_behind_steady(bool v_next) { // the same when every tile exists
    const int pk = 2 * (2 - kSNK), pv = 2 * (1 - kSNV) + 1;
    int p = pk > pv ? pk : pv;
    if (v_next && pv + 2 > p) p = pv + 2;
    return -1 - p;
}
__device__ __forceinline__ int sp_wrap(int x, int m) { return x >= m ? x - m : x; } // x < 2 m

#ifdef BZ_PF_TIMING
// Diagnostic build: every workgroup leaves the shader clock at a few points of its life in bz_pf_wg (read
// through bz_pf_wg_table); the library proper compiles none of it.
constexpr int kPftMaxWg = 32768;
__device__ unsigned long long bz_pf_wg[kPftMaxWg * 8];
#define BZ_PF_WG(k) do { __builtin_amdgcn_sched_barrier(0); pft[k] = __builtin_amdgcn_s_memtime(); __builtin_amdgcn_sched_barrier(0); } while (0)
#else
#define BZ_PF_WG(k) do { } while (0)
#endif
#ifdef BZ_PF_PHASES
// Diagnostic build on top of BZ_PF_TIMING: the first and the last wave of every workgroup add up, over their
// steady-state iterations, the shader clock spent in each part of an iteration (bz_pf_ph, read through
// bz_pf_phase_table).  Reading the clock waits for the wave's outstanding LDS reads, so the parts are a little
// longer than in the library proper.
__device__ unsigned long long bz_pf_ph[kPftMaxWg * 2 * 8];
#define BZ_PF_PH_START() do { __builtin_amdgcn_sched_barrier(0); ph_last = __builtin_amdgcn_s_memtime(); __builtin_amdgcn_sched_barrier(0); } while (0)
#define BZ_PF_PH(k) do { __builtin_amdgcn_sched_barrier(0); const unsigned long long t_ = __builtin_amdgcn_s_memtime(); ph[k] += t_ - ph_last; ph_last = t_; __builtin_amdgcn_sched_barrier(0); } while (0)
#else
#define BZ_PF_PH_START() do { } while (0)
#define BZ_PF_PH(k) do { } while (0)
#endif

// bf16 has two ways through the second contraction (the 8-bit significand of a bf16 probability alone would eat
// the error budget).  SPLIT_P: the probabilities enter it as head + tail of bf16, two matrix instructions per step.
// Otherwise (V_F16): the V tiles are widened to f16 in LDS, in place, one tile ahead of their use (each wave its
// quarter of the tile), the probabilities are packed as f16 and the second contraction runs on the f16
// instruction, one per step.  The widening is exact for |v| in f16's range (2^-24 .. 65504; smaller values round
// to f16 subnormals or zero, larger ones become infinite), which is why SPLIT_P stays selectable.
template <bool BF16, bool SPLIT_P, bool ROPE_Q>
__global__ __launch_bounds__(256, 2) void prefill_kernel(PrefillArgs a, const char* __restrict__ q_ptr,
                                                            const char* __restrict__ k_ptr,
                                                            const char* __restrict__ v_ptr) {
    constexpr bool V_F16 = BF16 && !SPLIT_P;
    using M = PfMma<BF16>;            // q, k, the first contraction and the output
    using MP = PfMma<BF16 && !V_F16>; // the probabilities and the second contraction
    constexpr bool QSCALED = ROPE_Q; // q carries sm_scale * log2(e)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
#ifdef BZ_PF_TIMING
#ifdef BZ_PF_PHASES
    unsigned long long ph[6] = {0, 0, 0, 0, 0, 0}, ph_last = 0;
#endif
    unsigned long long pft[8];
    pft[0] = __builtin_amdgcn_s_memtime();
    pft[7] = __builtin_amdgcn_s_memrealtime();
#endif

    const PrefillItem it = a.items[blockIdx.x];
    if (it.len <= 0) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int head = it.head;
    const int Hq = (int)a.num_qo_heads, Hkv = (int)a.num_kv_heads;
    const int kvh = head / (Hq / Hkv);
    const int qn = lane & 31, h = lane >> 5;
    // Lq q rows attend to L K/V rows (L >= Lq); q row i of the request sits at position off + i: it sees, when
    // causal, the tokens up to that position, and is rotated by that position.
    const int L = it.kv_len, Lq = it.len, off = L - Lq;
    const int wave_q_lo = it.q0 + 32 * wv;
    const int q_pos = wave_q_lo + qn;
    const int kv_limit = a.causal ? min(L, off + it.q0 + kBM) : L; // tokens any row of this workgroup can see
    const int n = (kv_limit + kSN - 1) / kSN;                      // tiles of the job
    // tiles this wave computes (causal: up to the diagonal tile of its last row; none for rows past the end of the
    // request); t_diag: the first tile in which one of its rows may have to be masked
    const int n_w = wave_q_lo >= Lq ? 0 : (a.causal ? min(n, (off + wave_q_lo + 31) / kSN + 1) : n);
    const int t_diag = a.causal ? (off + wave_q_lo) / kSN : 0x7fffffff;
    const int kv_max = a.causal ? min(off + q_pos, L - 1) : L - 1; // last token this row may see

    // ---- global -> LDS staging: wave wv moves rows 8wv .. 8wv+7 of a tile, two instructions of four 256-byte
    // rows each for K and for V (chunk XOR patterns: see the kernel's header)
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    const int r4 = lane >> 4, p16 = lane & 15;
    const uint32_t row_stride = (uint32_t)Hkv * 256u;
    uint32_t kcol[2], kfast[2], vfast[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) kcol[i] = (uint32_t)((p16 ^ ((8 * wv + 4 * i + r4) & 15)) * 16);
    const uint32_t vcol = (uint32_t)((p16 ^ BZ_VSWZ(r4)) * 16);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        kfast[i] = (uint32_t)(4 * i + r4) * row_stride + kcol[i] - (uint32_t)(i * 1024);
        vfast[i] = (uint32_t)(4 * i + r4) * row_stride + vcol - (uint32_t)(i * 1024);
    }
    const size_t kv_row0 = ((size_t)it.kv0 * Hkv + kvh) * 256; // byte offset of the request's first K/V row
    const char* const k_wave = k_ptr + kv_row0 + (size_t)(8 * wv) * row_stride;
    const char* const v_wave = v_ptr + kv_row0 + (size_t)(8 * wv) * row_stride;
    const uint32_t m0_wave = lds0 + (uint32_t)(8 * wv * 256);
    const size_t tile_stride = (size_t)kSN * row_stride;
    // a whole tile inside the request: one wave-uniform base, lane constants for the rest
    auto issue_k_fast = [&](int t, int slot) __attribute__((always_inline)) {
        lds_direct_load16x2(k_wave + (size_t)t * tile_stride, kfast[0], kfast[1], m0_wave + (uint32_t)(slot * kSTile));
    };
    auto issue_v_fast = [&](int t, int slot) __attribute__((always_inline)) {
        lds_direct_load16x2(v_wave + (size_t)t * tile_stride, vfast[0], vfast[1], m0_wave + (uint32_t)((kSNK + slot) * kSTile));
    };
    auto issue_k = [&](int t, int slot) __attribute__((always_inline)) {
        if ((t + 1) * kSN <= L) {
            issue_k_fast(t, slot);
        } else { // rows past the end of the request re-read its last row (masked later)
            const char* base = k_ptr + kv_row0 + (size_t)t * tile_stride;
            const uint32_t m0 = m0_wave + (uint32_t)(slot * kSTile);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int row = min(t * kSN + 8 * wv + 4 * i + r4, L - 1) - t * kSN;
                lds_direct_load16(base, (uint32_t)row * row_stride + kcol[i], m0 + i * 1024);
            }
        }
    };
    auto issue_v = [&](int t, int slot) __attribute__((always_inline)) {
        if ((t + 1) * kSN <= L) {
            issue_v_fast(t, slot);
        } else {
            const char* base = v_ptr + kv_row0 + (size_t)t * tile_stride;
            const uint32_t m0 = m0_wave + (uint32_t)((kSNK + slot) * kSTile);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int row = min(t * kSN + 8 * wv + 4 * i + r4, L - 1) - t * kSN;
                lds_direct_load16(base, (uint32_t)row * row_stride + vcol, m0 + i * 1024);
            }
        }
    };
    // ---- Q rows as B operands: lane (q, h) holds q[q][16*ks + 8*h .. +7], ks = 0..7.  The
    // loads of the q rows and of the angles go first, the tile copies of the prologue behind them; the rotation
    // is done while the copies travel.
    uint4 qreg[8];
    uint4 cs[ROPE_Q ? 16 : 1];
    {
        const size_t qtok = (size_t)it.tok0 + (size_t)min(q_pos, Lq - 1);
        const char* qrow = q_ptr + (qtok * Hq + head) * 256;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qreg[ks] = sp_load16(qrow + ks * 32 + h * 16);
        if constexpr (ROPE_Q) {
            // d = 16 ks + 8 h + e (ks < 4) pairs with d + 64, which this lane holds at step ks + 4.  The table is
            // laid out couple of pairs by couple of pairs, so the 32 rows of a half-wave read 512 consecutive bytes
            // per load.
            const float4* tab = a.rope_table + (off + min(q_pos, Lq - 1));
#pragma unroll
            for (int e = 0; e < 16; ++e) cs[e] = sp_load16(tab + (size_t)(8 * (e >> 2) + 4 * h + (e & 3)) * a.rope_pitch);
        }
    }
    int copies = 0; // tile copies issued so far
    if (L >= kSNK * kSN) {
        // the common case: the first tiles all exist and are whole (kv_limit >= 128 as well, so n >= 4)
#pragma unroll
        for (int i = -kSNK; i < 0; ++i) {
            issue_k_fast(i + kSNK, i + kSNK);
            if (i + kSNV - 1 >= 0) issue_v_fast(i + kSNV - 1, i + kSNV - 1);
        }
        copies = kSNK + kSNV - 1;
        sp_wait_copies(kSNK + kSNV - 1); // the q rows (and the angles) are here
    } else {
#pragma unroll
        for (int i = -kSNK; i < 0; ++i) {
            if (i + kSNK < n) { issue_k(i + kSNK, i + kSNK); ++copies; }
            if (i + kSNV - 1 >= 0 && i + kSNV - 1 < n) { issue_v(i + kSNV - 1, i + kSNV - 1); ++copies; }
        }
        sp_wait_copies(copies);
    }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) sp_loads_arrived(qreg[ks]);
    if constexpr (ROPE_Q) {
#pragma unroll
        for (int e = 0; e < 16; ++e) sp_loads_arrived(cs[e]);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint4 cw = cs[4 * ks + w]; // pairs i = 16 ks + 8 h + 2 w, i + 1
                const float2 c0 = make_float2(__uint_as_float(cw.x), __uint_as_float(cw.y));
                const float2 c1 = make_float2(__uint_as_float(cw.z), __uint_as_float(cw.w));
                const uint32_t xw = pf_u4(qreg[ks], w), yw = pf_u4(qreg[ks + 4], w);
                float x0, y0, x1, y1;
                rope_pair(M::lo(xw), M::lo(yw), c0.x, c0.y, x0, y0);
                rope_pair(M::hi(xw), M::hi(yw), c1.x, c1.y, x1, y1);
                // (the softmax scale rides on the one rounding of the rotated row, see the kernel's header: the
                // table holds cos and sin times sm_scale * log2(e))
                pf_u4(qreg[ks], w) = M::pack2(x0, x1);
                pf_u4(qreg[ks + 4], w) = M::pack2(y0, y1);
            }
    }

    // Operand reads.  K: lane (row qn, half h) needs chunk 2 ks + h of its row for step ks, which sits at position
    // (2 ks + h) ^ (qn % 16); V, through the transposing read: chunk 4 db + zl' of its row for d block db (see
    // the kernel's header).  One address register per step / d block (complete LDS addresses inside slot 0); the slot and
    // the token offsets of the V operands go into the instruction's offset field where they are compile-time constants.
    uint32_t koff[8], voff[4];
    {
        const int y = h ^ (qn & 15);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            koff[ks] = lds0 + (uint32_t)(qn * 256 + (((2 * ks) ^ y) * 16));
            asm volatile("" : "+v"(koff[ks])); // keep the sum: the compiler would rebuild it at every use
        }
        const int srow = (lane & 15) >> 2;
        const int zl = ((((lane >> 4) & 1) << 1) | ((lane & 3) >> 1)) ^ BZ_VSWZ(srow);
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            voff[db] = lds0 + (uint32_t)(kSNK * kSTile + (4 * h + srow) * 256 + ((((db << 2)) ^ zl) * 16) + (lane & 1) * 8);
            asm volatile("" : "+v"(voff[db]));
        }
    }
    uint4 kring[4], vring[4]; // operands of the matrix instructions, read four instructions ahead of their use
    typedef uint32_t __attribute__((ext_vector_type(4))) pf_u32x4;
    // (these issue the reads; the first use of a register waits for it.  `soff`: byte offset of the tile's slot)
    auto read_k = [&](uint4& dst, uint32_t soff, int ks) __attribute__((always_inline)) {
        const pf_u32x4 r = *reinterpret_cast<const pf_u32x4 __attribute__((address_space(3)))*>(
            (const unsigned char __attribute__((address_space(3)))*)(uintptr_t)(koff[ks]) + soff);
        dst = make_uint4(r.x, r.y, r.z, r.w);
    };
    // operand i = 4 st + db of the second contraction (tokens 16 st .., d block db): two reads, rows +0 and +8
    auto read_v = [&](uint4& dst, uint32_t soff, int i) __attribute__((always_inline)) {
        typedef pf_s16x4 __attribute__((address_space(3)))* lds_s16x4_ptr;
        const unsigned char __attribute__((address_space(3)))* vb =
            (const unsigned char __attribute__((address_space(3)))*)(uintptr_t)(voff[i & 3]) + soff + (i >> 2) * 16 * 256;
        const pf_s16x4 t0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(vb));
        const pf_s16x4 t1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(vb + 8 * 256));
        const uint2 w0 = __builtin_bit_cast(uint2, t0), w1 = __builtin_bit_cast(uint2, t1);
        dst = make_uint4(w0.x, w0.y, w1.x, w1.y);
    };
    // V_F16: this wave's quarter of the V tile in `slot` (the rows it copied), bf16 -> f16 in place
    auto widen_v = [&](int slot) __attribute__((always_inline)) {
        typedef pf_u32x4 __attribute__((address_space(3)))* lds_u32x4_ptr;
        unsigned char __attribute__((address_space(3)))* base =
            (unsigned char __attribute__((address_space(3)))*)(uintptr_t)(m0_wave + (uint32_t)((kSNK + slot) * kSTile)) + lane * 16;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            pf_u32x4 r = *(lds_u32x4_ptr)(base + i * 1024);
#pragma unroll
            for (int w = 0; w < 4; ++w)
                r[w] = PfMma<false>::pack2(__uint_as_float(r[w] << 16), __uint_as_float(r[w] & 0xffff0000u));
            *(lds_u32x4_ptr)(base + i * 1024) = r;
        }
    };
    auto k_at = [&](int slot) __attribute__((always_inline)) { return (uint32_t)(slot * kSTile); };
    auto v_at = [&](int slot) __attribute__((always_inline)) { return (uint32_t)(slot * kSTile); };

    // ---- softmax state (one reference maximum per row, moved only when it has to be: see the kernel's header)
    float m_run = 0.f, l_run = 0.f; // l_run: this lane's half of the row sum
    pf_f32x16 cinit;
#pragma unroll
    for (int i = 0; i < 16; ++i) cinit[i] = 0.f;
    pf_f32x16 acc[4]; // O^T: block db covers d = 32*db .. +31; element 4b+r is d = 32*db + 8b + 4h + r
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][i] = 0.f;
    pf_f32x16 s[2];     // scores of two tiles in flight: tile t lives in s[t % 2]
    uint4 pa[2], pb[2]; // P^T operands of the two 16-token steps of a tile (head, and tail when SPLIT_P)
    float psum = 0.f;

    auto mask_tile = [&](int t, pf_f32x16& sc) __attribute__((always_inline)) {
        // element 4b+r of a score block is token 32t + 8b + 4h + r
        if (t >= t_diag || (t + 1) * kSN > L) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int kv = t * kSN + 8 * (i >> 2) + 4 * h + (i & 3);
                sc[i] = kv > kv_max ? -INFINITY : sc[i];
            }
        }
    };
    auto exp_of = [&](float x, float shift) __attribute__((always_inline)) {
        return __builtin_amdgcn_exp2f(QSCALED ? x - shift : (x - shift) * a.sm_scale_log2);
    };
    // elements 2i, 2i+1 -> word i%4 of operand i/4.  The row sum takes the probabilities as they enter the second
    // contraction (rounded to the storage type; head + tail when SPLIT_P), one instruction per packed word.
    auto take_pair = [&](float p0, float p1, int i) __attribute__((always_inline)) {
        const uint32_t hw = MP::pack2_here(p0, p1);
        pf_u4(pa[i >> 2], i & 3) = hw;
        psum = MP::add_pair(hw, psum);
        if (SPLIT_P) {
            const uint32_t tw = MP::pack2_here(p0 - MP::lo(hw), p1 - MP::hi(hw));
            pf_u4(pb[i >> 2], i & 3) = tw;
            psum = MP::add_pair(tw, psum);
        }
    };
    // The first half of an iteration: scores of the next tile into s[PAR ^ 1] (QK) from K at k1 (steps 0..3 are in
    // the ring), probabilities of this tile from s[PAR] (EX), first V operands of this tile (at vj) into the ring.
    // The exponentials of step i are consumed in step i + 1 (their latency is longer than one instruction).
    auto first_half = [&](auto par_c, auto qk_c, auto ex_c, uint32_t k1, uint32_t vj) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value;
        constexpr bool QK = decltype(qk_c)::value, EX = decltype(ex_c)::value;
        float e0 = 0.f, e1 = 0.f;
        if (EX) psum = 0.f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (QK) s[PAR ^ 1] = M::run(kring[i & 3], qreg[i], i == 0 ? cinit : s[PAR ^ 1]);
            if (i < 4) read_k(kring[i], k1, i + 4);
            else read_v(vring[i - 4], vj, i - 4);
            if (EX) {
                const float n0 = exp_of(s[PAR][2 * i], 0.f), n1 = exp_of(s[PAR][2 * i + 1], 0.f);
                if (i > 0) take_pair(e0, e1, i - 1);
                e0 = n0;
                e1 = n1;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (EX) take_pair(e0, e1, 7);
        __builtin_amdgcn_sched_barrier(0);
    };
    // The second half: O += V^T P^T (PV), the rest of V (at vj) and the first K operands of the tile after the next
    // (at k2) into the rings
    auto second_half = [&](auto pv_c, uint32_t vj, uint32_t k2) __attribute__((always_inline)) {
        constexpr bool PV = decltype(pv_c)::value;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (PV) {
                acc[i & 3] = MP::run(vring[i & 3], pa[i >> 2], acc[i & 3]);
                if (SPLIT_P) acc[i & 3] = MP::run(vring[i & 3], pb[i >> 2], acc[i & 3]);
            }
            if (i < 4) read_v(vring[i], vj, i + 4);
            else read_k(kring[i - 4], k2, i - 4);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // the reference maximum has to move (some score of tile j is 15 or more above it): rare, wave-uniform
    auto move_maximum = [&](pf_f32x16& cur, pf_f32x16& next) __attribute__((always_inline)) {
        float tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, cur[i]);
        tmax = lane_max_xor32(tmax);
        const float shift = fmaxf(tmax, 0.f);
        const float alpha = __builtin_amdgcn_exp2f(QSCALED ? -shift : -shift * a.sm_scale_log2);
        m_run += shift;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[db][i] *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            cinit[i] = -m_run;
            next[i] -= shift; // the next tile's scores were taken against the old reference
        }
        psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) take_pair(exp_of(cur[2 * i], shift), exp_of(cur[2 * i + 1], shift), i);
    };

    // ---- prologue: scores of tile 0 set the reference maximum, the ring takes the first K operands of tile 1.
    // The copies were issued in the order K0 | K1 V0 | K2 V1 | K3 V2 (those that exist).
    BZ_PF_WG(1);
    sp_wait_copies(copies - 1); // K0 has landed
    sp_barrier();
    BZ_PF_WG(2);
    {
        uint4 k0[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) read_k(k0[i], k_at(0), i);
        if (n_w > 0) {
#pragma unroll
            for (int i = 0; i < 8; ++i) s[0] = M::run(k0[i], qreg[i], i == 0 ? cinit : s[0]);
            mask_tile(0, s[0]);
            float tmax = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[0][i]);
            tmax = lane_max_xor32(tmax); // finite: token 0 is visible to every row
            m_run = tmax;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                s[0][i] -= tmax;
                cinit[i] = -tmax;
            }
        }
        sp_wait_copies(max(copies - (V_F16 ? 3 : 2), 0)); // K1 has landed (if there is one); V_F16: V0 as well
        sp_barrier();
#pragma unroll
        for (int i = 0; i < 4; ++i) read_k(kring[i], k_at(1 % kSNK), i);
        if (V_F16) widen_v(0);
    }
    BZ_PF_WG(3);

    // ---- the steady state: every tile touched exists, is whole and needs no mask.  SL = j % 4 is the slot of
    // K(j) and of V(j), a compile-time constant (the loop is unrolled by four), so that LDS addresses are one
    // register plus an immediate and the copies' LDS targets are constants as well.
    const char* k_next = k_wave + (size_t)kSNK * tile_stride;       // K(j + kSNK)
    const char* v_next = v_wave + (size_t)(kSNV - 1) * tile_stride; // V(j + kSNV - 1)
    auto full = [&](int j, auto par_c, auto sl_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value, SL = decltype(sl_c)::value;
        BZ_PF_PH_START();
        sp_wait_copies(sp_copies_behind_steady(V_F16)); // K(j+2) and V(j) have landed (V_F16: V(j+1) too)
        BZ_PF_PH(0);
        sp_barrier();
        BZ_PF_PH(1);
        lds_direct_load16x2(k_next, kfast[0], kfast[1], m0_wave + (uint32_t)(SL * kSTile));
        lds_direct_load16x2(v_next, vfast[0], vfast[1], m0_wave + (uint32_t)((kSNK + (SL + kSNV - 1) % kSNV) * kSTile));
        k_next += tile_stride;
        v_next += tile_stride;
        if (V_F16) widen_v((SL + 1) % kSNV); // V(j+1), first read after the next barrier
        BZ_PF_PH(2);
        first_half(par_c, std::true_type{}, std::true_type{}, k_at((SL + 1) % kSNK), v_at(SL));
        BZ_PF_PH(3);
        if (__any(!(psum < 32768.0f))) move_maximum(s[PAR], s[PAR ^ 1]);
        l_run += psum;
        second_half(std::true_type{}, v_at(SL), k_at((SL + 2) % kSNK));
        BZ_PF_PH(4);
    };
    // ---- the same with every condition checked (the slots are still compile-time constants: j % 4 == SL).  The operand
    // reads are issued by every wave, also one that has nothing to compute, so that the registers have one definition
    // per iteration.
    auto generic = [&](int j, auto par_c, auto sl_c) __attribute__((always_inline)) {
        constexpr int PAR = decltype(par_c)::value, SL = decltype(sl_c)::value;
        const bool has_cur = j < n_w, has_next = j + 1 < n_w;
        sp_wait_copies(sp_copies_behind(j, n, V_F16));
        sp_barrier();
        if (j + kSNK < n) issue_k(j + kSNK, SL);
        if (j + kSNV - 1 < n) issue_v(j + kSNV - 1, (SL + kSNV - 1) % kSNV);
        if (V_F16 && j + 1 < n) widen_v((SL + 1) % kSNV);
        const uint32_t k1 = k_at((SL + 1) % kSNK), k2 = k_at((SL + 2) % kSNK);
        if (has_next) first_half(par_c, std::true_type{}, std::true_type{}, k1, v_at(SL));
        else first_half(par_c, std::false_type{}, std::true_type{}, k1, v_at(SL)); // (harmless without a tile: p of stale scores, never used)
        if (has_cur) {
            if (__any(!(psum < 32768.0f))) move_maximum(s[PAR], s[PAR ^ 1]);
            l_run += psum;
            if (has_next) mask_tile(j + 1, s[PAR ^ 1]);
            second_half(std::true_type{}, v_at(SL), k2);
        } else {
            second_half(std::false_type{}, v_at(SL), k2);
        }
    };
    // full needs: tiles j .. j+2 computed by this wave, tile j+1 unmasked, and the tiles it copies whole and in range
    const int j_full = min(min(n_w - 2, t_diag - 1), min(L / kSN, n) - kSNK);
    const std::integral_constant<int, 0> c0{};
    const std::integral_constant<int, 1> c1{};
    const std::integral_constant<int, 2> c2{};
    const std::integral_constant<int, 3> c3{};
    int j = 0;
    for (; j + 3 < j_full; j += 4) {
        full(j, c0, c0);
        full(j + 1, c1, c1);
        full(j + 2, c0, c2);
        full(j + 3, c1, c3);
    }
    BZ_PF_WG(4);
    // the rest (j is a multiple of four): the last tiles of the job, the diagonal ones and everything ragged.  Nested,
    // not one condition after the other: a tile's registers are then defined on one path only.
    for (; j < n; j += 4) {
        generic(j, c0, c0);
        if (j + 1 < n) {
            generic(j + 1, c1, c1);
            if (j + 2 < n) {
                generic(j + 2, c0, c2);
                if (j + 3 < n) generic(j + 3, c1, c3);
            }
        }
    }
    sp_barrier(); // nobody reads a tile any more: the epilogue takes their place
    BZ_PF_WG(5);

    // ---- epilogue: normalise, transpose the wave's 32 x 128 block through LDS (8 KiB per wave, 16-byte chunk c of
    // row r at c ^ (r % 16)), store whole rows
    const float l_row = lane_sum_xor32(l_run);
    const float inv_l = l_row > 0.f ? 1.0f / l_row : 0.f;
    unsigned char* o_lds = smem + wv * (32 * 256);
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t w0 = M::pack2(acc[db][4 * b] * inv_l, acc[db][4 * b + 1] * inv_l);
            const uint32_t w1 = M::pack2(acc[db][4 * b + 2] * inv_l, acc[db][4 * b + 3] * inv_l);
            const int chunk = 4 * db + b; // d = 32 db + 8 b + 4 h .. +3: bytes 64 db + 16 b + 8 h
            *reinterpret_cast<uint2*>(o_lds + qn * 256 + ((chunk ^ (qn & 15)) * 16) + 8 * h) = make_uint2(w0, w1);
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int ps = 0; ps < 8; ++ps) {
        const int row = 4 * ps + (lane >> 4);
        const int pos = wave_q_lo + row;
        if (pos < Lq) {
            const uint4 v = *reinterpret_cast<const uint4*>(o_lds + row * 256 + (((lane & 15) ^ (row & 15)) * 16));
            char* orow = (char*)a.out + (((size_t)it.tok0 + pos) * Hq + head) * 256;
            *reinterpret_cast<uint4*>(orow + (lane & 15) * 16) = v;
        }
    }
#ifdef BZ_PF_PHASES
    if ((wv == 0 || wv == 3) && lane == 0 && blockIdx.x < kPftMaxWg) {
        unsigned long long* dst = bz_pf_ph + ((size_t)blockIdx.x * 2 + (wv == 3 ? 1 : 0)) * 8;
        for (int i = 0; i < 5; ++i) dst[i] = ph[i];
        dst[5] = (unsigned long long)max(j_full, 0) / 4 * 4; // steady-state iterations of this wave
    }
#endif
#ifdef BZ_PF_TIMING
    if (tid == 0 && blockIdx.x < kPftMaxWg) {
        pft[6] = __builtin_amdgcn_s_memtime();
        // HW_ID: wave 3:0, simd 5:4, pipe 7:6, cu 11:8, sh 12, se 15:13 (...); XCC_ID: 3:0
        unsigned hw = 0, xcc = 0;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        bz_pf_wg[blockIdx.x * 8 + 0] = ((unsigned long long)n << 32) | (unsigned)max(j_full, 0);
        bz_pf_wg[blockIdx.x * 8 + 2] = ((unsigned long long)(xcc & 15) << 32) | hw; // (replaces the K0-landed stamp)
        for (int i = 1; i < 7; ++i) if (i != 2) bz_pf_wg[blockIdx.x * 8 + i] = pft[i] - pft[0];
        bz_pf_wg[blockIdx.x * 8 + 7] = ((__builtin_amdgcn_s_memrealtime() - pft[7]) << 40) | (pft[7] & 0xffffffffffull);
    }
#endif
}

// ---- in-place RoPE of ragged rows, one token per workgroup (used when the caller asks the attention call itself to
// rotate).  K rows sit at their index inside the request; q rows, when a request has more K/V rows than q rows, at
// that index plus the difference (`longer`: the K/V index of the batch, given for q rows only).
struct RopeRaggedArgs {
    void* rows;
    const int32_t* indptr; // ragged index of `rows`
    const int32_t* longer; // nullptr, or the ragged index whose request lengths set the offset of the positions
    uint32_t batch_size, num_heads;
    RopeFreqs freqs;
};

template <typename T>
__global__ __launch_bounds__(256) void rope_ragged_kernel(RopeRaggedArgs a) {
    __shared__ float s_cos[64], s_sin[64];
    __shared__ int s_b;
    const int ntok = a.indptr[a.batch_size];
    const int tok = blockIdx.x;
    if (tok >= ntok) return;
    if (threadIdx.x == 0) {
        int lo = 0, hi = (int)a.batch_size;
        while (hi - lo > 1) {
            const int mid = (lo + hi) / 2;
            if (a.indptr[mid] <= tok) lo = mid; else hi = mid;
        }
        s_b = lo;
    }
    __syncthreads();
    int pos = tok - a.indptr[s_b];
    if (a.longer) pos += (a.longer[s_b + 1] - a.longer[s_b]) - (a.indptr[s_b + 1] - a.indptr[s_b]);
    if (threadIdx.x < 64) {
        float s, c;
        sincosf((float)pos * a.freqs.f[threadIdx.x], &s, &c);
        s_cos[threadIdx.x] = c;
        s_sin[threadIdx.x] = s;
    }
    __syncthreads();
    const int lane8 = threadIdx.x & 7; // 8 lanes per row: 8 low-half and the 8 matching high-half elements each
    for (int r = threadIdx.x >> 3; r < (int)a.num_heads; r += 32) {
        T* row = reinterpret_cast<T*>(a.rows) + ((size_t)tok * a.num_heads + r) * 128;
        Vec8<T> lo, hi;
        lo.load(row + lane8 * 8);
        hi.load(row + 64 + lane8 * 8);
        float x[8], y[8];
        lo.to_float(x);
        hi.to_float(y);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float c = s_cos[lane8 * 8 + e], s = s_sin[lane8 * 8 + e];
            float xr, yr;
            rope_pair(x[e], y[e], c, s, xr, yr);
            x[e] = xr;
            y[e] = yr;
        }
        lo.from_float(x);
        hi.from_float(y);
        lo.store(row + lane8 * 8);
        hi.store(row + 64 + lane8 * 8);
    }
}

// cos / sin table for the q rotation inside the attention kernel: table[i / 2][pos] = (cos, sin) of pair i (even)
// and of pair i + 1 at that position, each times `scale` (sm_scale * log2(e): the rotated rows come out scaled)
__global__ __launch_bounds__(256) void rope_table_kernel(float4* table, uint32_t positions, uint32_t pitch, RopeFreqs freqs,
                                                         float scale) {
    const uint32_t pos = blockIdx.x * 256 + threadIdx.x, i = 2 * blockIdx.y;
    if (pos >= positions) return;
    float s0, c0, s1, c1;
    sincosf((float)pos * freqs.f[i], &s0, &c0);
    sincosf((float)pos * freqs.f[i + 1], &s1, &c1);
    table[(size_t)blockIdx.y * pitch + pos] = make_float4(c0 * scale, s0 * scale, c1 * scale, s1 * scale);
}

static inline size_t pf_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

} // namespace bz

using namespace bz;

extern "C" bz_prefill_plan_t* bz_prefill_plan_create(void) {
    return reinterpret_cast<bz_prefill_plan_t*>(new (std::nothrow) PrefillPlan());
}

extern "C" int bz_prefill_plan_set_bf16_mode(bz_prefill_plan_t* plan_, int mode) {
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    if (!p || (mode != BZ_PREFILL_BF16_WIDEN_V && mode != BZ_PREFILL_BF16_HEAD_TAIL)) return BZ_ERR_BAD_ARG;
    p->bf16_head_tail = mode == BZ_PREFILL_BF16_HEAD_TAIL;
    return 0;
}

extern "C" int bz_prefill_plan_set_timing_events(bz_prefill_plan_t* plan_, void* start_event, void* stop_event) {
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    if (!p || ((start_event == nullptr) != (stop_event == nullptr))) return BZ_ERR_BAD_ARG;
    p->time_start = (hipEvent_t)start_event;
    p->time_stop = (hipEvent_t)stop_event;
    return 0;
}

extern "C" void bz_prefill_plan_destroy(bz_prefill_plan_t* plan_) {
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    if (!p) return;
    if (p->upload_done) {
        (void)hipEventSynchronize(p->upload_done);
        (void)hipEventDestroy(p->upload_done);
    }
    if (p->staging) (void)hipHostFree(p->staging);
    delete p;
}

// Pure host work: the job list of a ragged batch into p->h_items.
static int build_prefill_items(PrefillPlan* p, const int32_t* qo_indptr_h, const int32_t* kv_indptr_h,
                               uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim) {
    if (!p || !qo_indptr_h || !kv_indptr_h) return BZ_ERR_BAD_ARG;
    if (num_kv_heads == 0 || num_qo_heads % num_kv_heads) return BZ_ERR_BAD_ARG;
    p->planned = false;
    if (head_dim != 128) return BZ_ERR_UNSUPPORTED;
    // The reference passes the same array twice (src/layer/attn.h:175-187).  With two arrays a request has q rows
    // for its last tokens only (a chunk of a prompt whose earlier K/V rows are given again): at least as many
    // K/V rows as q rows.
    if (qo_indptr_h[0] != 0 || kv_indptr_h[0] != 0) return BZ_ERR_BAD_ARG;
    for (uint32_t b = 0; b < batch_size; ++b) {
        if (kv_indptr_h[b + 1] < kv_indptr_h[b]) return BZ_ERR_BAD_ARG;
        if (kv_indptr_h[b + 1] - kv_indptr_h[b] < qo_indptr_h[b + 1] - qo_indptr_h[b]) return BZ_ERR_UNSUPPORTED;
    }
    // One entry per workgroup, in launch order.  Workgroups are dealt round-robin to the 8 XCDs, each
    // with its own L2, so launch index i runs on XCD i % 8.  Every (request, kv head) unit is given to one
    // XCD as a run of consecutive jobs: its q tiles (of all q heads of the group) then execute together on
    // that XCD and share the unit's K/V (up to 2 MiB for 4096 tokens) through that L2 instead of each
    // fetching it from HBM.  Units go to the XCDs in turn, longest requests first, so every XCD gets the same
    // mix of work.
    for (uint32_t b = 0; b < batch_size; ++b)
        if (qo_indptr_h[b + 1] < qo_indptr_h[b]) return BZ_ERR_BAD_ARG;
    std::vector<uint32_t> order(batch_size);
    for (uint32_t b = 0; b < batch_size; ++b) order[b] = b;
    std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { // (a tile's work goes with the K/V length)
        return kv_indptr_h[x + 1] - kv_indptr_h[x] > kv_indptr_h[y + 1] - kv_indptr_h[y];
    });
    constexpr int kXcd = 8;
    std::vector<PrefillItem> per_xcd[kXcd];
    uint32_t pair = 0;
    // Grouped-query attention: the q heads of one kv head read the same K/V, so they go to one XCD
    // together, tile by tile (the same K/V tiles are then in flight for all of them at once) -- as long
    // as that leaves at least two units of work per XCD; otherwise the group is cut into parts.
    const uint32_t G = num_qo_heads / num_kv_heads;
    uint32_t live = 0;
    for (uint32_t b = 0; b < batch_size; ++b) live += qo_indptr_h[b + 1] > qo_indptr_h[b];
    uint32_t parts = 1;
    while (parts < G && (G % parts || (uint64_t)live * num_kv_heads * parts < 2 * kXcd)) ++parts;
    const uint32_t per_part = G / parts;
    // A workgroup and the one that shares its compute unit (32 launch positions later in the XCD's list)
    // step through their units in the same order, so jobs of the same size meet and their phases coincide:
    // both wait for copies at once, both want the matrix cores at once.  Every second unit of an XCD's list
    // therefore runs its tiles from the first (fewest keys) to the last, which pairs long jobs with short
    // ones.  The last two units of a list, and lists too short for the order to matter, keep most-keys-first,
    // so that the XCD's work does not end on its longest jobs.
    const uint32_t units_per_xcd = live * num_kv_heads * parts / kXcd; // (rounded down)
    for (uint32_t b : order) {
        const int32_t len = qo_indptr_h[b + 1] - qo_indptr_h[b];
        if (len == 0) continue;
        const int32_t last_q0 = (len - 1) / kBM * kBM;
        for (uint32_t unit = 0; unit < num_kv_heads * parts; ++unit, ++pair) {
            const uint32_t nth = pair / kXcd; // the unit's place in its XCD's list
            const bool ascending = (nth & 1) && units_per_xcd >= 6 && nth + 2 < units_per_xcd;
            for (int32_t qi = last_q0; qi >= 0; qi -= kBM)
                for (uint32_t g = 0; g < per_part; ++g)
                    per_xcd[pair % kXcd].push_back({qo_indptr_h[b], len, ascending ? last_q0 - qi : qi,
                                                    (int32_t)(unit * per_part + g), kv_indptr_h[b],
                                                    kv_indptr_h[b + 1] - kv_indptr_h[b], {0, 0}});
        }
    }
    size_t longest = 0;
    for (auto& v : per_xcd) longest = std::max(longest, v.size());
    std::vector<PrefillItem>& items = p->h_items;
    items.assign(longest * kXcd, PrefillItem{0, 0, 0, 0, 0, 0, {0, 0}});
    for (int x = 0; x < kXcd; ++x)
        for (size_t k = 0; k < per_xcd[x].size(); ++k) items[k * kXcd + x] = per_xcd[x][k];
    return 0;
}

extern "C" int bz_prefill_plan_workspace(bz_prefill_plan_t* plan_, const int32_t* qo_indptr_h, const int32_t* kv_indptr_h,
                                         uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads,
                                         uint32_t head_dim, size_t* float_buffer_bytes, size_t* int_buffer_bytes) {
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    const int rc = build_prefill_items(p, qo_indptr_h, kv_indptr_h, batch_size, num_qo_heads, num_kv_heads, head_dim);
    if (rc) return rc;
    if (float_buffer_bytes) { // the angle table of the q rotation: 512 bytes per position of the longest request
        int32_t longest = 0;
        for (uint32_t b = 0; b < batch_size; ++b) longest = std::max(longest, kv_indptr_h[b + 1] - kv_indptr_h[b]);
        *float_buffer_bytes = (size_t)longest * 512;
    }
    if (int_buffer_bytes) *int_buffer_bytes = pf_align_up(p->h_items.size() * sizeof(PrefillItem), 256);
    return 0;
}

extern "C" int bz_prefill_plan_host_schedule(const bz_prefill_plan_t* plan_, const int32_t** data, size_t* num_records,
                                             uint32_t* ints_per_record) {
    const PrefillPlan* p = reinterpret_cast<const PrefillPlan*>(plan_);
    if (!p || !data || !num_records || !ints_per_record) return BZ_ERR_BAD_ARG;
    *data = (const int32_t*)p->h_items.data();
    *num_records = p->h_items.size();
    *ints_per_record = sizeof(PrefillItem) / 4;
    return 0;
}

extern "C" int bz_prefill_plan(bz_prefill_plan_t* plan_, void* float_buffer, size_t float_buffer_bytes,
                               void* int_buffer, size_t int_buffer_bytes, const int32_t* qo_indptr_h,
                               const int32_t* kv_indptr_h, uint32_t batch_size, uint32_t num_qo_heads,
                               uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_size, void* stream) {
    (void)page_size;
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    if (!p || !int_buffer) return BZ_ERR_BAD_ARG;
    const int rc0 = build_prefill_items(p, qo_indptr_h, kv_indptr_h, batch_size, num_qo_heads, num_kv_heads, head_dim);
    if (rc0) return rc0;
    const std::vector<PrefillItem>& items = p->h_items;
    const size_t bytes = pf_align_up(items.size() * sizeof(PrefillItem), 256);
    if (bytes > int_buffer_bytes) return BZ_ERR_WORKSPACE;
    hipStream_t s = (hipStream_t)stream;
    if (!p->upload_done) BZ_CHECK_HIP(hipEventCreateWithFlags(&p->upload_done, hipEventDisableTiming));
    else BZ_CHECK_HIP(hipEventSynchronize(p->upload_done));
    if (bytes > p->staging_bytes) {
        if (p->staging) BZ_CHECK_HIP(hipHostFree(p->staging));
        p->staging = nullptr;
        p->staging_bytes = 0;
        const size_t want = std::max<size_t>(pf_align_up(bytes * 2, 4096), 1 << 16);
        BZ_CHECK_HIP(hipHostMalloc(&p->staging, want, hipHostMallocDefault));
        p->staging_bytes = want;
    }
    if (bytes) {
        memset(p->staging, 0, bytes);
        memcpy(p->staging, items.data(), items.size() * sizeof(PrefillItem));
        BZ_CHECK_HIP(hipMemcpyAsync(int_buffer, p->staging, bytes, hipMemcpyHostToDevice, s));
    }
    BZ_CHECK_HIP(hipEventRecord(p->upload_done, s));
    p->items_d = (const PrefillItem*)int_buffer;
    p->num_items = (uint32_t)items.size();
    p->batch_size = batch_size; p->num_qo_heads = num_qo_heads; p->num_kv_heads = num_kv_heads;
    p->head_dim = head_dim;
    p->total_tokens = (uint32_t)qo_indptr_h[batch_size];
    p->total_kv_tokens = (uint32_t)kv_indptr_h[batch_size];
    p->max_len = 0;
    for (uint32_t b = 0; b < batch_size; ++b)
        p->max_len = std::max<uint32_t>(p->max_len, (uint32_t)(kv_indptr_h[b + 1] - kv_indptr_h[b]));
    // the float workspace holds the angle table of the q rotation when it has room for it (512 bytes per position)
    p->rope_table = (float_buffer && (size_t)p->max_len * 512 <= float_buffer_bytes && (uintptr_t)float_buffer % 16 == 0)
                        ? (float*)float_buffer : nullptr;
    p->planned = true;
    return 0;
}

template <bool BF16, bool SPLIT_P, bool ROPE_Q>
static int launch_prefill(const PrefillPlan* p, const PrefillArgs& a, const void* q, const void* k, const void* v,
                             hipStream_t s) {
    auto kern = prefill_kernel<BF16, SPLIT_P, ROPE_Q>;
    static std::atomic<uint64_t> attr_done{0};
    int dev = 0;
    BZ_CHECK_HIP(hipGetDevice(&dev));
    const uint64_t bit = 1ull << (dev & 63);
    if (!(attr_done.load(std::memory_order_relaxed) & bit)) {
        BZ_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kSLds));
        attr_done.fetch_or(bit, std::memory_order_relaxed);
    }
    if (p->time_start) BZ_CHECK_HIP(hipEventRecord(p->time_start, s));
    hipLaunchKernelGGL(kern, dim3(p->num_items), dim3(256), kSLds, s, a, (const char*)q, (const char*)k, (const char*)v);
    BZ_LAUNCH_CHECK();
    if (p->time_stop) BZ_CHECK_HIP(hipEventRecord(p->time_stop, s));
    return 0;
}

#ifdef BZ_PF_PHASES
extern "C" int bz_pf_phase_table(unsigned long long* host, size_t count) {
    if (count > sizeof(bz_pf_ph) / 8) count = sizeof(bz_pf_ph) / 8;
    BZ_CHECK_HIP(hipMemcpyFromSymbol(host, HIP_SYMBOL(bz_pf_ph), count * 8, 0, hipMemcpyDeviceToHost));
    return 0;
}
#endif
#ifdef BZ_PF_TIMING
// copies the table of the diagnostic build to the host: per workgroup 8 values (see prefill_kernel)
extern "C" int bz_pf_wg_table(unsigned long long* host, size_t count) {
    if (count > sizeof(bz_pf_wg) / 8) count = sizeof(bz_pf_wg) / 8;
    BZ_CHECK_HIP(hipMemcpyFromSymbol(host, HIP_SYMBOL(bz_pf_wg), count * 8, 0, hipMemcpyDeviceToHost));
    return 0;
}
#endif

extern "C" int bz_batch_prefill_ragged(bz_prefill_plan_t* plan_, void* q, const int32_t* qo_indptr, void* k, void* v,
                                       const int32_t* kv_indptr, void* out, int dtype, uint32_t batch_size,
                                       uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim, int causal,
                                       int rope_mode, float rope_theta, float sm_scale, void* stream) {
    PrefillPlan* p = reinterpret_cast<PrefillPlan*>(plan_);
    if (!p || !q || !k || !v || !out || !qo_indptr || !kv_indptr) return BZ_ERR_BAD_ARG;
    if (!p->planned) return BZ_ERR_NOT_PLANNED;
    if (batch_size != p->batch_size || num_qo_heads != p->num_qo_heads || num_kv_heads != p->num_kv_heads ||
        head_dim != p->head_dim)
        return BZ_ERR_BAD_ARG;
    if (dtype != BZ_F16 && dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED;
    if (rope_mode < BZ_ROPE_NONE || rope_mode > BZ_ROPE_FULL) return BZ_ERR_BAD_ARG;
    if (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16) return BZ_ERR_BAD_ARG;
    hipStream_t s = (hipStream_t)stream;
    // q is rotated in registers inside the attention kernel (angles from a table in the float workspace) and
    // stays as it is in memory; k, which every q tile of a request reads, is rotated once, in place, first.
    bool rope_q = rope_mode != BZ_ROPE_NONE;
    if (rope_mode != BZ_ROPE_NONE) {
        const float theta = rope_theta > 0.f ? rope_theta : 1e4f;
        const RopeFreqs freqs = make_rope_freqs(128, theta);
        if (p->rope_table && p->num_items > 0) {
            // (every call: the workspace may be shared with other handlers between calls, calls may change streams,
            // and a captured call must replay its own fill; a few microseconds)
            const float scale = (sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)head_dim)) * 1.4426950408889634f;
            hipLaunchKernelGGL(rope_table_kernel, dim3((p->max_len + 255) / 256, 32), dim3(256), 0, s, (float4*)p->rope_table,
                               p->max_len, p->max_len, freqs, scale);
            BZ_LAUNCH_CHECK();
        }
        auto rotate_rows = [&](void* rows, const int32_t* indptr, const int32_t* longer, uint32_t heads, uint32_t tokens) {
            RopeRaggedArgs ra;
            ra.rows = rows; ra.indptr = indptr; ra.longer = longer;
            ra.batch_size = batch_size; ra.num_heads = heads;
            ra.freqs = freqs;
            if (tokens == 0) return;
            if (dtype == BZ_F16) hipLaunchKernelGGL((rope_ragged_kernel<f16_t>), dim3(tokens), dim3(256), 0, s, ra);
            else hipLaunchKernelGGL((rope_ragged_kernel<bf16_t>), dim3(tokens), dim3(256), 0, s, ra);
        };
        if (rope_mode == BZ_ROPE_FULL) rotate_rows(k, kv_indptr, nullptr, num_kv_heads, p->total_kv_tokens);
        if (!p->rope_table) rotate_rows(q, qo_indptr, kv_indptr, num_qo_heads, p->total_tokens); // no room for the table
        BZ_LAUNCH_CHECK();
        rope_q = p->rope_table != nullptr;
    }
    if (p->num_items == 0) return 0; // no q rows in the batch (K, if the call was to rotate it, has been rotated)
    PrefillArgs a;
    a.out = out;
    a.items = p->items_d;
    a.rope_table = (const float4*)p->rope_table;
    a.rope_pitch = p->max_len;
    a.num_qo_heads = num_qo_heads; a.num_kv_heads = num_kv_heads;
    a.causal = causal ? 1 : 0;
    if (!(sm_scale > 0.f)) sm_scale = 1.0f / sqrtf((float)head_dim);
    a.sm_scale_log2 = sm_scale * 1.4426950408889634f;
    if (rope_q) {
        if (dtype == BZ_F16) return launch_prefill<false, false, true>(p, a, q, k, v, s);
        if (p->bf16_head_tail) return launch_prefill<true, true, true>(p, a, q, k, v, s);
        return launch_prefill<true, false, true>(p, a, q, k, v, s);
    }
    if (dtype == BZ_F16) return launch_prefill<false, false, false>(p, a, q, k, v, s);
    if (p->bf16_head_tail) return launch_prefill<true, true, false>(p, a, q, k, v, s);
    return launch_prefill<true, false, false>(p, a, q, k, v, s);
}
