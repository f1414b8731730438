// MFMA paged decode for gfx950 (head_dim 128, page_size a multiple of 16, f16/bf16 KV, up to 16
// query heads per kv head).  One wave64 per workgroup walks a list of "pieces" (contiguous runs of
// 32-token tiles of one (sequence, kv head)) that the host planner balanced over the wave slots
// of the chip, so every K and V byte is read once and shared by all query heads of the group.
//
// Per 32-token tile, with S^T = K Q^T so that the MFMA result layout of the scores is already the
// A-operand layout of the P V product (no shuffles between the two contractions):
//   K rows   : global -> VGPR, 16 B per lane, used directly as MFMA A operands (contraction over d)
//   V rows   : global -> VGPR -> LDS (row stride 288 B), read back with the transposing LDS load
//              (ds_read_b64_tr_b16) as MFMA B operands (contraction over tokens)
//   softmax  : online, 8 scores per lane, row max / sum over the 4 lane groups with two shuffles
// The loads of tile t+1 are issued before the arithmetic of tile t.
#include <cmath>

#include "bz_common.hpp"
#include "bz_decode_plan.hpp"

namespace bz {

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
    const MfmaPiece* pieces;
    const int32_t* piece_ptr;
    float* part_o;   // [num_partials][16][128]
    float* part_lse; // [num_partials][16]
    uint64_t stride_page, stride_n, stride_h; // elements
    uint32_t page_size, num_qo_heads, group;
    int rope_q;
    float sm_scale_log2;
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
        return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
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

// The read-only inputs are separate __restrict__ parameters so that wave-uniform reads of the page
// table and of the schedule go through the scalar unit.
template <bool BF16, typename OT, bool ROPE_Q>
__global__ __launch_bounds__(64, 2) void decode_mfma_kernel(MfmaDecodeArgs a, const char* __restrict__ q_ptr,
                                                            const char* __restrict__ k_data,
                                                            const char* __restrict__ v_data,
                                                            const int32_t* __restrict__ indices,
                                                            const int32_t* __restrict__ indptr,
                                                            const int32_t* __restrict__ last_page_len,
                                                            const MfmaPiece* __restrict__ pieces,
                                                            const int32_t* __restrict__ piece_ptr) {
    using M = Mma<BF16>;
    __shared__ __attribute__((aligned(16))) unsigned char v_lds[kTileTok * kVRowBytes];

    const int lane = threadIdx.x;
    const int n = lane & 15; // query head (scores) / d column (output) / token row (K operand)
    const int j = lane >> 4; // lane group: which 8-wide slice of the MFMA contraction
    const int P = (int)a.page_size;
    const size_t row_bytes = (size_t)a.stride_n * 2;
    const int G = (int)a.group;

    const int p_begin = piece_ptr[blockIdx.x], p_end = piece_ptr[blockIdx.x + 1];
    for (int pi = p_begin; pi < p_end; ++pi) {
        const MfmaPiece pc = pieces[pi];
        const int b = pc.seq, kvh = pc.kvh;
        const int ip0 = indptr[b];
        const int npages = indptr[b + 1] - ip0;
        const int seq_len = (npages - 1) * P + last_page_len[b];
        const int tok_end = min(pc.tile_end * kTileTok, seq_len);
        const size_t head_bytes = (size_t)kvh * a.stride_h * 2;

        // ---- Q as MFMA B operand: lane (head n, group j) holds q[head][32*ks + 8*j .. +7], ks = 0..3.
        // With in-kernel RoPE the rotated q is split into a storage-precision head and tail (q = hi + lo)
        // and both are contracted, so the rotation costs no precision.
        uint4 qhi[4], qlo[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) { qhi[ks] = make_uint4(0, 0, 0, 0); qlo[ks] = make_uint4(0, 0, 0, 0); }
        if (n < G) {
            const char* qrow = q_ptr + ((size_t)b * a.num_qo_heads + (size_t)kvh * G + n) * 256;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qhi[ks] = *reinterpret_cast<const uint4*>(qrow + ks * 64 + j * 16);
            if (ROPE_Q) {
                const float pos = (float)(seq_len - 1);
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) { // dims d = 32ks+8j+e pair with d+64, held at ks+2
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        float x[2] = {M::unpack_lo(u4(qhi[ks], w)), M::unpack_hi(u4(qhi[ks], w))};
                        float y[2] = {M::unpack_lo(u4(qhi[ks + 2], w)), M::unpack_hi(u4(qhi[ks + 2], w))};
                        float xr[2], yr[2];
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            float s, c;
                            sincosf(pos * a.freqs.f[32 * ks + 8 * j + 2 * w + e], &s, &c);
                            xr[e] = x[e] * c - y[e] * s;
                            yr[e] = y[e] * c + x[e] * s;
                        }
                        const uint32_t xh = M::pack2(xr[0], xr[1]), yh = M::pack2(yr[0], yr[1]);
                        u4(qhi[ks], w) = xh;
                        u4(qhi[ks + 2], w) = yh;
                        u4(qlo[ks], w) = M::pack2(xr[0] - M::unpack_lo(xh), xr[1] - M::unpack_hi(xh));
                        u4(qlo[ks + 2], w) = M::pack2(yr[0] - M::unpack_lo(yh), yr[1] - M::unpack_hi(yh));
                    }
                }
            }
        }

        float m_run = -INFINITY, l_run = 0.f;
        f32x4_t acc[8];
#pragma unroll
        for (int d = 0; d < 8; ++d) acc[d] = f32x4_t{0.f, 0.f, 0.f, 0.f};

        // Page ids of the two 16-token subtiles of a tile.  A tile may reach past the last page of the
        // sequence: the lookup stays in bounds (last page, slot 0) and the tokens are masked later.
        // The ids are fetched one tile ahead of the loads that need them.
        int pid[2];
        auto load_pids = [&](int tile) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                int pg = (tile * kTileTok + 16 * u) / P;
                pg = pg < npages ? pg : npages - 1;
                pid[u] = indices[ip0 + pg];
            }
        };
        auto subtile_base = [&](int tile, int u) -> size_t {
            const int tok = tile * kTileTok + 16 * u;
            const int slot0 = (tok / P < npages) ? tok % P : 0;
            return ((size_t)pid[u] * a.stride_page + (size_t)slot0 * a.stride_n) * 2 + head_bytes;
        };

        uint4 kreg[2][4], vreg[8];
        auto issue_loads = [&](int tile) {
            const size_t b0 = subtile_base(tile, 0), b1 = subtile_base(tile, 1);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                kreg[0][ks] = *reinterpret_cast<const uint4*>(k_data + b0 + (size_t)n * row_bytes + ks * 64 + j * 16);
                kreg[1][ks] = *reinterpret_cast<const uint4*>(k_data + b1 + (size_t)n * row_bytes + ks * 64 + j * 16);
            }
#pragma unroll
            for (int w = 0; w < 8; ++w) { // rows 4w..4w+3 of the tile, 16 lanes x 16 B per row
                const int row = 4 * w + j;
                const size_t bb = (row < 16) ? b0 : b1;
                vreg[w] = *reinterpret_cast<const uint4*>(v_data + bb + (size_t)(row & 15) * row_bytes + n * 16);
            }
        };

        load_pids(pc.tile_begin);
        issue_loads(pc.tile_begin);
        load_pids(pc.tile_begin + 1);
        for (int t = pc.tile_begin; t < pc.tile_end; ++t) {
            const int tile_tok0 = t * kTileTok;
            const bool ragged = tile_tok0 + kTileTok > tok_end; // wave-uniform
            __syncthreads(); // transposed reads of the previous tile are done before V is overwritten
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                uint4 v = vreg[w];
                if (ragged && tile_tok0 + 4 * w + j >= tok_end) v = make_uint4(0, 0, 0, 0); // 0 * garbage must be 0
                *reinterpret_cast<uint4*>(v_lds + (4 * w + j) * kVRowBytes + n * 16) = v;
            }
            uint4 kcur[2][4];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) kcur[u][ks] = kreg[u][ks];
            if (t + 1 < pc.tile_end) {
                issue_loads(t + 1);
                load_pids(t + 2);
            }

            // ---- scores: S^T[token][head], lane (head n, group j) gets tokens 16u + 4j + r
            f32x4_t s[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                s[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) s[u] = M::run(kcur[u][ks], qhi[ks], s[u]);
                if (ROPE_Q) {
#pragma unroll
                    for (int ks = 0; ks < 4; ++ks) s[u] = M::run(kcur[u][ks], qlo[ks], s[u]);
                }
            }
            float tmax = -INFINITY;
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = s[u][r] * a.sm_scale_log2;
                    if (ragged && tile_tok0 + 16 * u + 4 * j + r >= tok_end) v = -INFINITY;
                    s[u][r] = v;
                    tmax = fmaxf(tmax, v);
                }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            const float m_new = fmaxf(m_run, tmax);      // finite: every tile holds at least one live token
            const float alpha = exp2f(m_run - m_new);    // 0 on the first tile (m_run = -inf)
            // The probabilities enter the second contraction as a storage-precision head plus tail
            // (p = hi + lo, two MFMAs per block): the matrix cores cost nothing here and the result
            // keeps fp32-level accuracy instead of the 8 to 11 bits of a single rounded operand.
            float psum = 0.f;
            uint4 pa, pb;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const float p0 = exp2f(s[u][0] - m_new), p1 = exp2f(s[u][1] - m_new);
                const float p2 = exp2f(s[u][2] - m_new), p3 = exp2f(s[u][3] - m_new);
                psum += (p0 + p1) + (p2 + p3);
                const uint32_t h01 = M::pack2(p0, p1), h23 = M::pack2(p2, p3);
                u4(pa, 2 * u) = h01;
                u4(pa, 2 * u + 1) = h23;
                u4(pb, 2 * u) = M::pack2(p0 - M::unpack_lo(h01), p1 - M::unpack_hi(h01));
                u4(pb, 2 * u + 1) = M::pack2(p2 - M::unpack_lo(h23), p3 - M::unpack_hi(h23));
            }
            psum += __shfl_xor(psum, 16, 64);
            psum += __shfl_xor(psum, 32, 64);
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
            __syncthreads(); // V tile visible to every lane
            // ---- O[head][d] += P[head][tok] V[tok][d], eight 16-wide d blocks
#pragma unroll
            for (int d = 0; d < 8; ++d) {
                uint4 vb;
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const unsigned char* src =
                        v_lds + (16 * u + 4 * j + (n >> 2)) * kVRowBytes + d * 32 + (n & 3) * 8;
                    const s16x4_t tr = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4_t __attribute__((address_space(3)))*)(src));
                    const uint2 w = __builtin_bit_cast(uint2, tr);
                    u4(vb, 2 * u) = w.x;
                    u4(vb, 2 * u + 1) = w.y;
                }
                acc[d] = M::run(pa, vb, acc[d]);
                acc[d] = M::run(pb, vb, acc[d]);
            }
        }

        // ---- epilogue: normalise and write the final rows, or the split-K partial
        const float inv_l = l_run > 0.f ? 1.0f / l_run : 0.f;
        const float lse2 = l_run > 0.f ? m_run + log2f(l_run) : -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = 4 * j + i;
            const float il = __shfl(inv_l, head, 64);
            if (head < G) {
                const int hq = kvh * G + head;
                if (pc.partial < 0) {
                    OT* orow = reinterpret_cast<OT*>(a.out) + ((size_t)b * a.num_qo_heads + hq) * 128;
#pragma unroll
                    for (int d = 0; d < 8; ++d) orow[d * 16 + n] = StoreCvt<OT>::from(acc[d][i] * il);
                } else {
                    float* prow = a.part_o + ((size_t)pc.partial * 16 + head) * 128;
#pragma unroll
                    for (int d = 0; d < 8; ++d) prow[d * 16 + n] = acc[d][i] * il;
                }
            }
        }
        if (j == 0 && n < G) {
            if (pc.partial < 0) {
                if (a.lse) a.lse[(size_t)b * a.num_qo_heads + kvh * G + n] = lse2 * 0.6931471805599453f;
            } else {
                a.part_lse[(size_t)pc.partial * 16 + n] = lse2;
            }
        }
    }
}

// Combine the partials of one split (sequence, kv head): o = sum_i o_i 2^(lse_i - M) / sum_i 2^(lse_i - M).
template <typename OT>
__global__ __launch_bounds__(128) void decode_mfma_combine_kernel(const MfmaCombine* combos, const float* part_o,
                                                                  const float* part_lse, void* out, float* lse,
                                                                  uint32_t num_qo_heads, uint32_t G) {
    const MfmaCombine c = combos[blockIdx.x];
    const uint32_t g = blockIdx.y, d = threadIdx.x;
    float M = -INFINITY;
    for (int i = 0; i < c.count; ++i) M = fmaxf(M, part_lse[(size_t)(c.first + i) * 16 + g]);
    float wsum = 0.f, o = 0.f;
    for (int i = 0; i < c.count; ++i) {
        const float li = part_lse[(size_t)(c.first + i) * 16 + g];
        const float w = (li == -INFINITY) ? 0.f : exp2f(li - M);
        wsum += w;
        o += w * part_o[((size_t)(c.first + i) * 16 + g) * 128 + d];
    }
    o = wsum > 0.f ? o / wsum : 0.f;
    const size_t hq = (size_t)c.seq * num_qo_heads + (size_t)c.kvh * G + g;
    reinterpret_cast<OT*>(out)[hq * 128 + d] = StoreCvt<OT>::from(o);
    if (lse && d == 0) lse[hq] = (M + log2f(wsum)) * 0.6931471805599453f;
}

struct DecodeArgs; // general-kernel argument block (bz_decode.hip); only its scalar fields are forwarded here

template <bool BF16, typename OT>
static int launch_mfma(const DecodePlan* p, const MfmaDecodeArgs& a, hipStream_t s) {
    if (a.rope_q)
        hipLaunchKernelGGL((decode_mfma_kernel<BF16, OT, true>), dim3(p->mfma_slots), dim3(64), 0, s, a,
                           (const char*)a.q, a.k_data, a.v_data, a.indices, a.indptr, a.last_page_len, a.pieces,
                           a.piece_ptr);
    else
        hipLaunchKernelGGL((decode_mfma_kernel<BF16, OT, false>), dim3(p->mfma_slots), dim3(64), 0, s, a,
                           (const char*)a.q, a.k_data, a.v_data, a.indices, a.indptr, a.last_page_len, a.pieces,
                           a.piece_ptr);
    BZ_LAUNCH_CHECK();
    if (p->mfma_combos > 0) {
        hipLaunchKernelGGL((decode_mfma_combine_kernel<OT>), dim3(p->mfma_combos, a.group), dim3(128), 0, s,
                           p->mfma_combos_d, a.part_o, a.part_lse, a.out, a.lse, a.num_qo_heads, a.group);
        BZ_LAUNCH_CHECK();
    }
    return 0;
}

int decode_fast_path(const DecodePlan* p, const void* q, void* out, float* lse, int q_dtype, int out_dtype,
                     int rope_mode, float sm_scale_log2, const RopeFreqs& freqs, const bz_paged_kv_t* kv,
                     uint32_t num_qo_heads, hipStream_t s) {
    if (!p->mfma_ok || p->mfma_slots == 0) return BZ_ERR_UNSUPPORTED;
    if (kv->kv_dtype != q_dtype || rope_mode == BZ_ROPE_FULL) return BZ_ERR_UNSUPPORTED;
    if ((kv->stride_n * 2) % 16 || (kv->stride_h * 2) % 16 || (kv->stride_page * 2) % 16) return BZ_ERR_UNSUPPORTED;
    if (((uintptr_t)kv->k_data | (uintptr_t)kv->v_data | (uintptr_t)q) % 16) return BZ_ERR_UNSUPPORTED;
    MfmaDecodeArgs a;
    a.q = q; a.out = out; a.lse = lse;
    a.k_data = (const char*)kv->k_data; a.v_data = (const char*)kv->v_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.pieces = p->mfma_pieces_d; a.piece_ptr = p->mfma_piece_ptr_d;
    a.part_o = p->mfma_part_o; a.part_lse = p->mfma_part_lse;
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.page_size = kv->page_size; a.num_qo_heads = num_qo_heads; a.group = num_qo_heads / kv->num_kv_heads;
    a.rope_q = rope_mode == BZ_ROPE_Q_ONLY;
    a.sm_scale_log2 = sm_scale_log2;
    a.freqs = freqs;
    if (q_dtype == BZ_BF16)
        return out_dtype == BZ_F32 ? launch_mfma<true, float>(p, a, s) : launch_mfma<true, bf16_t>(p, a, s);
    return out_dtype == BZ_F32 ? launch_mfma<false, float>(p, a, s) : launch_mfma<false, f16_t>(p, a, s);
}

} // namespace bz
