// Paged-KV batch decode attention for gfx950: host-side plan (split-K segmentation), the
// general VALU kernel (any layout / dtype / RoPE mode) and the split-K combine.
// Replaces src/kernel/attention_decode.cu and the decode half of flashinfer_types.cu of the
// BlitzScale worker.
#include <cmath>
#include <algorithm>
#include <mutex>
#include <vector>
#include <new>

#include <type_traits>

#include "bz_common.hpp"
#include "bz_decode_plan.hpp"

namespace bz {

// ------------------------------------------------------------------------------------------
// General kernel.  One workgroup of 256 lanes per (segment, kv head).  A row of D elements is
// covered by D/8 lanes holding 8 elements each, so the workgroup walks TOK = 256/(D/8) tokens
// per pass; every token slot keeps its own online-softmax state (m, l, acc) for the G query
// heads that share the kv head, and the slots are merged once at the end.
// ------------------------------------------------------------------------------------------
template <typename KVT, int D> struct RowGeom {
    static constexpr int kLanes = D / 8;          // lanes per row
    static constexpr int kTok = 256 / kLanes;     // token slots per workgroup
    static constexpr int kTokPerWave = 64 / kLanes;
};

struct DecodeArgs {
    const void* q;
    void* out;
    float* lse;
    const char* k_data;
    const char* v_data;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    const int32_t* steps_ahead; // optional: the table is this many decode steps ahead of the present
    const DecodeSegment* segments;
    float* part_o;   // [num_partials][Hq][D]
    float* part_lse; // [num_partials][Hq]
    const float* k_scale;
    const float* v_scale;
    uint64_t stride_page, stride_n, stride_h;
    uint32_t page_size, num_qo_heads, num_kv_heads;
    uint32_t group_div; // workgroups per kv head: a group that is no instantiated size is split into equal parts
    int rope_mode;
    float sm_scale_log2; // sm_scale * log2(e)
    const float2* rope_table; // BZ_ROPE_FULL: (cos, sin) per [position][pair] or nullptr (angles computed on the fly)
    int rope_positions;       // positions the table holds: every slot of every page the plan lists
    RopeFreqs freqs;
};

// (cos, sin) of position * frequency i for positions [0, positions): the expression the kernels evaluate on the
// fly, evaluated once per plan instead of once per cached token, kv head and step.
__global__ __launch_bounds__(256) void decode_rope_table_kernel(float2* table, uint32_t positions, uint32_t pairs,
                                                                RopeFreqs freqs) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i >= positions * pairs) return;
    float s, c;
    sincosf((float)(i / pairs) * freqs.f[i % pairs], &s, &c);
    table[i] = make_float2(c, s);
}

// Sum over the N (8 or 16) consecutive lanes that share a token row, left in every one of them.  Row rotations
// and quad permutes of the DPP path (one full-rate instruction per step) where the lanes of a row are the 16
// lanes of a DPP row; an 8-lane row needs one cross-lane read for its upper and lower half.
template <int N> __device__ __forceinline__ float row_sum(float v) {
    auto dpp_add = [](float x, auto ctrl) {
        constexpr int C = decltype(ctrl)::value;
        return x + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), C, 0xF, 0xF, false));
    };
    if constexpr (N == 16) {
        v = dpp_add(v, std::integral_constant<int, 0x128>{}); // row_ror:8
        v = dpp_add(v, std::integral_constant<int, 0x124>{}); // row_ror:4
    } else {
        static_assert(N == 8, "rows of 8 or 16 lanes");
        v += __shfl_xor(v, 4, 64);
    }
    v = dpp_add(v, std::integral_constant<int, 0x4E>{}); // quad_perm [2,3,0,1]
    v = dpp_add(v, std::integral_constant<int, 0xB1>{}); // quad_perm [1,0,3,2]
    return v;
}

// TABLE: BZ_ROPE_FULL with the angles of the cached K rows taken from a.rope_table (an instantiation of its own,
// so that the registers the table rows travel through do not cost the other modes their occupancy).
template <typename QT, typename KVT, typename OT, int D, int G, bool TABLE = false>
__global__ __launch_bounds__(256) void decode_general_kernel(DecodeArgs a) {
    using Geo = RowGeom<KVT, D>;
    constexpr int LANES = Geo::kLanes;
    constexpr int TOK = Geo::kTok;
    constexpr int UNROLL = G == 8 ? 2 : 4; // tokens per lane slot and register set

    const DecodeSegment seg = a.segments[blockIdx.x];
    const int unit = blockIdx.y;                   // G consecutive q heads, all of one kv head
    const int kvh = unit / (int)a.group_div;
    const int b = seg.seq;
    const int tid = threadIdx.x;
    const int lane_in_row = tid % LANES; // which 8-element slice of the row
    const int slot = tid / LANES;        // token slot 0..TOK-1

    const int ahead = a.steps_ahead ? *a.steps_ahead : 0;
    const int ip0 = a.indptr[b];
    const int npages = a.indptr[b + 1] - ip0;
    const int seq_len = max((npages - 1) * (int)a.page_size + a.last_page_len[b] - max(ahead, 0), 0);
    const int tok_begin = seg.page_begin * (int)a.page_size;
    const int tok_end = min(seg.page_end * (int)a.page_size, seq_len);

    // ---- q for the G heads of this kv head, as fp32, pre-rotated if asked ----
    float q[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const size_t qoff = ((size_t)b * a.num_qo_heads + (size_t)unit * G + g) * D + lane_in_row * 8;
        Vec8<QT> qv;
        qv.load(reinterpret_cast<const QT*>(a.q) + qoff);
        qv.to_float(q[g]);
    }
    if (a.rope_mode != BZ_ROPE_NONE) {
        // partner slice holds the other half of each rotate-half pair
        const bool upper = lane_in_row >= LANES / 2;
        const float pos = (float)(seq_len - 1);
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float other = __shfl_xor(q[g][e], LANES / 2, 64);
                const int fi = (lane_in_row % (LANES / 2)) * 8 + e;
                float s, c;
                sincosf(pos * a.freqs.f[fi], &s, &c);
                float lo_r, hi_r; // this lane's element is x of its pair (lower half) or y (upper half)
                rope_pair(upper ? other : q[g][e], upper ? q[g][e] : other, c, s, lo_r, hi_r);
                q[g][e] = upper ? hi_r : lo_r;
            }
        }
    }
    const float kscale = (a.k_scale ? a.k_scale[kvh] : 1.0f) * a.sm_scale_log2;

    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
    }

    const size_t esz = sizeof(KVT);
    const size_t head_off = ((size_t)kvh * a.stride_h + (size_t)lane_in_row * 8) * esz;

    // BZ_ROPE_FULL rotates every cached K row at its own position.  Evaluating sincosf per element makes the
    // kernel compute-bound several times over, so the angles come from a table when the plan has room for one
    // (64 bytes per lane and token, fetched TU tokens ahead; the groups of eight q heads have no registers left
    // for that and keep the on-the-fly evaluation).
    constexpr int TU = G <= 2 ? 4 : 2;
    static_assert(!TABLE || G <= 4, "no registers for the table rows beside eight q heads");
    constexpr bool table_rope = TABLE;
    const float4* cs_lane = reinterpret_cast<const float4*>(a.rope_table) + (lane_in_row % (LANES / 2)) * 4;

    // Two register sets of UNROLL tokens per lane slot take turns: the loads of the next set go out before the
    // arithmetic of the present one.  They are issued whether or not the set has a live token (addresses are
    // clamped to a token of the segment): with the same number of loads behind a set on every path, the waits the
    // compiler derives for a set leave the other set's loads in flight.  (Not for single heads per workgroup,
    // whose occupancy the second set would cost.)
    struct TokSet {
        Vec8<KVT> kv[UNROLL], vv[UNROLL];
        bool valid[UNROLL];
        int jj[UNROLL];
    };
    auto issue = [&](int base, TokSet& S) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int j = base + u * TOK + slot;
            S.jj[u] = j;
            S.valid[u] = j < tok_end;
            const int jc = S.valid[u] ? j : tok_begin; // any in-range token: keeps the load legal
            const int64_t page = a.indices[ip0 + jc / (int)a.page_size];
            const size_t off =
                ((size_t)page * a.stride_page + (size_t)(jc % (int)a.page_size) * a.stride_n) * esz + head_off;
            S.kv[u].load_nt(a.k_data + off); // read once per launch (+2 to 3 % over plain loads)
            S.vv[u].load_nt(a.v_data + off);
        }
    };
    auto compute = [&](TokSet& S) __attribute__((always_inline)) {
        Vec8<KVT>(&kv)[UNROLL] = S.kv;
        Vec8<KVT>(&vv)[UNROLL] = S.vv;
        bool(&valid)[UNROLL] = S.valid;
        int(&jj)[UNROLL] = S.jj;
        float4 cs[TABLE ? TU : 1][4]; // (cos, sin) of this lane's eight pairs at the positions of TU tokens
        auto fetch_cs = [&](int u) {
            // (a sequence cannot be longer than its planned pages hold, which the table covers; the bound keeps the
            // read inside the table whatever the device-side lengths say)
            const int jc = min(valid[u] ? jj[u] : tok_begin, a.rope_positions - 1);
            const float4* row = cs_lane + (size_t)jc * (D / 4); // D/2 pairs of 8 bytes = D/4 float4 per position
#pragma unroll
            for (int i = 0; i < 4; ++i) cs[u % TU][i] = row[i];
        };
        if constexpr (TABLE) {
#pragma unroll
            for (int u = 0; u < TU; ++u) fetch_cs(u);
        }
        // Scores of the UNROLL tokens first (a token's row is spread over LANES lanes: products, then a sum across
        // the lanes of the row with DPP row rotations), then one softmax update per q head for all of them: one
        // maximum, one rescale of the accumulators per batch instead of per token, raw v_exp_f32.
        float sc_tok[UNROLL][G];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            float kf[8];
            kv[u].to_float(kf);
            if (a.rope_mode == BZ_ROPE_FULL) {
                const bool upper = lane_in_row >= LANES / 2;
                float cv[8], sv[8];
                if constexpr (TABLE) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float4 t = cs[u % TU][i];
                        cv[2 * i] = t.x; sv[2 * i] = t.y; cv[2 * i + 1] = t.z; sv[2 * i + 1] = t.w;
                    }
                    if (u + TU < UNROLL) fetch_cs(u + TU);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float other = __shfl_xor(kf[e], LANES / 2, 64);
                    const int fi = (lane_in_row % (LANES / 2)) * 8 + e;
                    float s, c;
                    if constexpr (TABLE) { c = cv[e]; s = sv[e]; }
                    else sincosf((float)jj[u] * a.freqs.f[fi], &s, &c);
                    float lo_r, hi_r;
                    rope_pair(upper ? other : kf[e], upper ? kf[e] : other, c, s, lo_r, hi_r);
                    kf[e] = upper ? hi_r : lo_r;
                }
            }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) s += q[g][e] * kf[e];
                s = row_sum<LANES>(s);
                sc_tok[u][g] = valid[u] ? s * kscale : -INFINITY;
            }
        }
        float vf[UNROLL][8];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) vv[u].to_float(vf[u]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float mx = m[g];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) mx = fmaxf(mx, sc_tok[u][g]);
            const float mref = fmaxf(mx, -1e30f); // finite also while nothing live has been seen: weights come out 0
            const float sc = __builtin_amdgcn_exp2f(m[g] - mref); // m = -inf before the first live token gives 0
            float p[UNROLL], psum = 0.f;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                p[u] = __builtin_amdgcn_exp2f(sc_tok[u][g] - mref); // -inf (no such token) gives 0
                psum += p[u];
            }
            l[g] = l[g] * sc + psum;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = acc[g][e] * sc;
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) t += p[u] * vf[u][e];
                acc[g][e] = t;
            }
            m[g] = mx;
        }
    };
    constexpr int STEP = TOK * UNROLL;
    if constexpr (G >= 2) {
        TokSet A, B;
        if (tok_begin < tok_end) issue(tok_begin, A);
        for (int base = tok_begin; base < tok_end; base += 2 * STEP) {
            issue(base + STEP, B);
            compute(A);
            issue(base + 2 * STEP, A);
            if (base + STEP < tok_end) compute(B);
        }
    } else {
        for (int base = tok_begin; base < tok_end; base += STEP) {
            TokSet A;
            issue(base, A);
            compute(A);
        }
    }

    // ---- merge the token slots: first inside the wave, then across the 4 waves through LDS ----
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int o = LANES; o < 64; o <<= 1) {
            const float mo = __shfl_xor(m[g], o, 64);
            const float lo = __shfl_xor(l[g], o, 64);
            const float mn = fmaxf(m[g], mo);
            const float sa = (m[g] == -INFINITY) ? 0.f : exp2f(m[g] - mn);
            const float sb = (mo == -INFINITY) ? 0.f : exp2f(mo - mn);
            l[g] = l[g] * sa + lo * sb;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float ao = __shfl_xor(acc[g][e], o, 64);
                acc[g][e] = acc[g][e] * sa + ao * sb;
            }
            m[g] = mn;
        }
    }
    __shared__ float sm_m[4][G];
    __shared__ float sm_l[4][G];
    __shared__ float sm_acc[4][G][D];
    const int wave = tid / 64, lane = tid % 64;
    if (lane < LANES) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (lane == 0) { sm_m[wave][g] = m[g]; sm_l[wave][g] = l[g]; }
#pragma unroll
            for (int e = 0; e < 8; ++e) sm_acc[wave][g][lane * 8 + e] = acc[g][e];
        }
    }
    __syncthreads();
    const float vscale = a.v_scale ? a.v_scale[kvh] : 1.0f;
    for (int idx = tid; idx < G * D; idx += 256) {
        const int g = idx / D, d = idx % D;
        float mm = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) mm = fmaxf(mm, sm_m[w][g]);
        float ll = 0.f, oo = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float sc = (sm_m[w][g] == -INFINITY) ? 0.f : exp2f(sm_m[w][g] - mm);
            ll += sm_l[w][g] * sc;
            oo += sm_acc[w][g][d] * sc;
        }
        const float o = (ll > 0.f) ? oo / ll * vscale : 0.f;
        const float lse2 = (ll > 0.f) ? mm + log2f(ll) : -INFINITY; // base-2 log-sum-exp of scaled logits
        const int hq = unit * G + g;
        if (seg.partial < 0) {
            reinterpret_cast<OT*>(a.out)[((size_t)b * a.num_qo_heads + hq) * D + d] = StoreCvt<OT>::from(o);
            if (a.lse && d == 0) a.lse[(size_t)b * a.num_qo_heads + hq] = lse2 * 0.6931471805599453f;
        } else {
            a.part_o[((size_t)seg.partial * a.num_qo_heads + hq) * D + d] = o;
            if (d == 0) a.part_lse[(size_t)seg.partial * a.num_qo_heads + hq] = lse2;
        }
    }
}

// ------------------------------------------------------------------------------------------
// Split-K combine: o = sum_i o_i 2^(lse_i - M) / sum_i 2^(lse_i - M) over the partial results of
// one sequence.  One workgroup of D lanes per (split sequence, q head).
// ------------------------------------------------------------------------------------------
template <typename OT>
__global__ void decode_combine_kernel(const DecodeCombine* combos, const float* part_o, const float* part_lse,
                                      void* out, float* lse, uint32_t num_qo_heads, uint32_t D) {
    const DecodeCombine c = combos[blockIdx.x];
    const uint32_t h = blockIdx.y, d = threadIdx.x;
    float M = -INFINITY;
    for (int i = 0; i < c.count; ++i) M = fmaxf(M, part_lse[(size_t)(c.first + i) * num_qo_heads + h]);
    float wsum = 0.f, o = 0.f;
    for (int i = 0; i < c.count; ++i) {
        const float li = part_lse[(size_t)(c.first + i) * num_qo_heads + h];
        const float w = (li == -INFINITY) ? 0.f : exp2f(li - M);
        wsum += w;
        o += w * part_o[((size_t)(c.first + i) * num_qo_heads + h) * D + d];
    }
    o = wsum > 0.f ? o / wsum : 0.f;
    reinterpret_cast<OT*>(out)[((size_t)c.seq * num_qo_heads + h) * D + d] = StoreCvt<OT>::from(o);
    if (lse && d == 0) lse[(size_t)c.seq * num_qo_heads + h] = (M + log2f(wsum)) * 0.6931471805599453f;
}

// zero rows of sequences with no pages (seq_len 0): the general kernel never visits them
template <typename OT>
__global__ void decode_zero_rows_kernel(const int32_t* empty_seqs, void* out, uint32_t row_elems) {
    const int b = empty_seqs[blockIdx.x];
    for (uint32_t i = threadIdx.x; i < row_elems; i += blockDim.x)
        reinterpret_cast<OT*>(out)[(size_t)b * row_elems + i] = StoreCvt<OT>::from(0.f);
}

// ------------------------------------------------------------------------------------------
// dispatch
// ------------------------------------------------------------------------------------------
template <typename QT, typename KVT, typename OT, int D>
static int launch_general_g(const DecodeArgs& a, int G, dim3 grid, hipStream_t s) {
    if constexpr (std::is_same<QT, KVT>::value) {
        if (a.rope_mode == BZ_ROPE_FULL && a.rope_table && G <= 4) { // angles from the table
            switch (G) {
                case 1: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 1, true>), grid, dim3(256), 0, s, a); break;
                case 2: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 2, true>), grid, dim3(256), 0, s, a); break;
                default: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 4, true>), grid, dim3(256), 0, s, a); break;
            }
            BZ_LAUNCH_CHECK();
            return 0;
        }
    }
    switch (G) {
        case 1: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 1>), grid, dim3(256), 0, s, a); break;
        case 2: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 2>), grid, dim3(256), 0, s, a); break;
        case 4: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 4>), grid, dim3(256), 0, s, a); break;
        case 8: hipLaunchKernelGGL((decode_general_kernel<QT, KVT, OT, D, 8>), grid, dim3(256), 0, s, a); break;
        default: return BZ_ERR_UNSUPPORTED;
    }
    BZ_LAUNCH_CHECK();
    return 0;
}

template <typename QT, typename KVT, typename OT>
static int launch_general_d(const DecodeArgs& a, int D, int G, dim3 grid, hipStream_t s) {
    if (D == 128) return launch_general_g<QT, KVT, OT, 128>(a, G, grid, s);
    if (D == 64) return launch_general_g<QT, KVT, OT, 64>(a, G, grid, s);
    return BZ_ERR_UNSUPPORTED;
}

template <typename QT, typename OT>
static int launch_general_kv(const DecodeArgs& a, int kv_dtype, int q_dtype, int D, int G, dim3 grid,
                             hipStream_t s) {
    if (kv_dtype == BZ_E4M3) return launch_general_d<QT, e4m3_t, OT>(a, D, G, grid, s);
    if (kv_dtype == q_dtype) return launch_general_d<QT, QT, OT>(a, D, G, grid, s);
    return BZ_ERR_UNSUPPORTED;
}

template <typename OT>
static void launch_combine(const DecodePlan* p, const float* part_o, const float* part_lse, void* out, float* lse,
                           uint32_t Hq, uint32_t D, hipStream_t s) {
    hipLaunchKernelGGL((decode_combine_kernel<OT>), dim3(p->num_combos, Hq), dim3(D), 0, s, p->combos_d, part_o,
                       part_lse, out, lse, Hq, D);
}
template <typename OT>
static void launch_zero(const DecodePlan* p, void* out, uint32_t row_elems, hipStream_t s) {
    hipLaunchKernelGGL((decode_zero_rows_kernel<OT>), dim3(p->num_empty), dim3(256), 0, s, p->empty_d, out, row_elems);
}

int decode_fast_path(const DecodePlan* p, const void* q, void* out, float* lse, int q_dtype, int out_dtype,
                     int rope_mode, float sm_scale_log2, const RopeFreqs& freqs, const bz_paged_kv_t* kv,
                     uint32_t num_qo_heads, const float* k_scale, const float* v_scale, float* part_o,
                     float* part_lse, bool step_mode, hipStream_t s); // bz_decode_mfma.hip

int decode_step_fast_path(const DecodePlan* p, const void* q, const void* k_new, const void* v_new, void* out,
                          float* lse, int q_dtype, int out_dtype, int rope, float sm_scale_log2,
                          const RopeFreqs& freqs, const bz_paged_kv_t* kv, uint32_t num_qo_heads, const float* k_scale,
                          const float* v_scale, hipStream_t s); // bz_decode_mfma.hip

// Where the split-K partial results of one call live: the plan's float workspace (bz_batch_decode) or the
// library's own device array (bz_batch_decode_noalloc).  The two kernels never run in the same call, so
// both pairs may point at the same memory.
struct PartialBufs {
    float *part_o, *part_lse;           // general kernel: [partials][Hq][D], [partials][Hq]
    float *mfma_part_o, *mfma_part_lse; // matrix-core kernel: [partials][16][128], [partials][16]
};

static int batch_decode_impl(DecodePlan* p, const void* q, int q_dtype, const bz_paged_kv_t* kv, void* out,
                             int out_dtype, uint32_t num_qo_heads, int rope_mode, float rope_theta, float sm_scale,
                             const float* k_scale, const float* v_scale, float* lse, const PartialBufs* bufs_or_null,
                             void* stream) {
    if (!p || !kv || !q || !out) return BZ_ERR_BAD_ARG;
    if (!p->planned) return BZ_ERR_NOT_PLANNED;
    // a table whose device pointers were cleared after the previous step (src/blitz/stub.h:1361-1363)
    if (!kv->k_data || !kv->v_data || !kv->indices || !kv->indptr || !kv->last_page_len) return BZ_ERR_BAD_ARG;
    if (kv->batch_size != p->batch_size || kv->page_size != p->page_size || kv->num_kv_heads != p->num_kv_heads ||
        kv->head_dim != p->head_dim || num_qo_heads != p->num_qo_heads)
        return BZ_ERR_BAD_ARG;
    if (q_dtype != BZ_F16 && q_dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED;
    if (out_dtype != q_dtype && out_dtype != BZ_F32) return BZ_ERR_UNSUPPORTED;
    if (kv->kv_dtype != q_dtype && kv->kv_dtype != BZ_E4M3) return BZ_ERR_UNSUPPORTED;
    if (num_qo_heads % kv->num_kv_heads) return BZ_ERR_BAD_ARG;
    if (rope_mode < BZ_ROPE_NONE || rope_mode > BZ_ROPE_FULL) return BZ_ERR_BAD_ARG;
    // 8-element vectors need rows that start on a vector boundary
    if (kv->stride_n % 8 || kv->stride_h % 8 || kv->stride_page % 8) return BZ_ERR_BAD_ARG;
    const int D = (int)kv->head_dim, G = (int)(num_qo_heads / kv->num_kv_heads);
    hipStream_t s = (hipStream_t)stream;
    if (p->batch_size == 0) return 0;
    const PartialBufs from_plan = {p->part_o, p->part_lse, p->mfma_part_o, p->mfma_part_lse};
    const PartialBufs& bufs = bufs_or_null ? *bufs_or_null : from_plan;

    DecodeArgs a;
    a.q = q; a.out = out; a.lse = lse;
    a.k_data = (const char*)kv->k_data; a.v_data = (const char*)kv->v_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.steps_ahead = kv->steps_ahead;
    a.segments = p->segments_d;
    a.part_o = bufs.part_o; a.part_lse = bufs.part_lse;
    a.k_scale = k_scale; a.v_scale = v_scale;
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.page_size = kv->page_size; a.num_qo_heads = num_qo_heads; a.num_kv_heads = kv->num_kv_heads;
    a.group_div = 1;
    a.rope_mode = rope_mode;
    a.rope_table = nullptr;
    a.rope_positions = 0;
    if (!(sm_scale > 0.f)) sm_scale = 1.0f / sqrtf((float)D);
    a.sm_scale_log2 = sm_scale * 1.4426950408889634f;
    a.freqs = make_rope_freqs(D, rope_theta > 0.f ? rope_theta : 1e4f);

    if (p->num_segments > 0) {
        int rc = BZ_ERR_UNSUPPORTED;
        if (!p->force_general)
            rc = decode_fast_path(p, q, out, lse, q_dtype, out_dtype, rope_mode, a.sm_scale_log2, a.freqs, kv,
                                  num_qo_heads, k_scale, v_scale, bufs.mfma_part_o, bufs.mfma_part_lse, false, s);
        if (rc == 0) {
            // the MFMA path brings its own combine; only empty sequences are left to do
            if (p->num_empty > 0) {
                const uint32_t row = num_qo_heads * D;
                if (out_dtype == BZ_F32) launch_zero<float>(p, out, row, s);
                else if (out_dtype == BZ_F16) launch_zero<f16_t>(p, out, row, s);
                else launch_zero<bf16_t>(p, out, row, s);
                BZ_LAUNCH_CHECK();
            }
            return 0;
        }
        if (rc == BZ_ERR_UNSUPPORTED) {
            // groups of 1, 2, 4 or 8 q heads per workgroup; any other group size is split into equal parts of
            // the largest of these that divides it (each part reads the K/V of its kv head again)
            int Gk = 8;
            while (G % Gk) Gk >>= 1;
            a.group_div = (uint32_t)(G / Gk);
            // kRoPELlama on a raw-K cache: the angle table behind the general partials of the plan's own float
            // workspace, when it fits (512 bytes per position at head_dim 128).  It is written by every call, on the
            // call's stream, in front of the kernel that reads it (a few microseconds): the workspace may be shared
            // with other handlers between calls, calls may change streams, and a captured call must replay its own
            // fill -- a table kept from an earlier call could be stale in each of these cases without any sign of it.
            if (rope_mode == BZ_ROPE_FULL && !bufs_or_null && p->max_seq_len > 0) {
                const size_t off = (p->general_part_bytes + 255) / 256 * 256;
                const uint32_t positions = (p->max_seq_len + p->page_size - 1) / p->page_size * p->page_size;
                const size_t tbytes = (size_t)positions * (size_t)(D / 2) * sizeof(float2);
                if (off + tbytes <= p->float_buffer_bytes) {
                    float2* table = reinterpret_cast<float2*>(reinterpret_cast<char*>(p->part_o) + off);
                    const uint32_t n = positions * (uint32_t)(D / 2);
                    hipLaunchKernelGGL(decode_rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, s, table, positions,
                                       (uint32_t)(D / 2), a.freqs);
                    BZ_LAUNCH_CHECK();
                    a.rope_table = table;
                    a.rope_positions = (int)positions;
                }
            }
            dim3 grid(p->num_segments, kv->num_kv_heads * a.group_div);
            if (p->time_start) BZ_CHECK_HIP(hipEventRecord(p->time_start, s));
            if (q_dtype == BZ_F16)
                rc = (out_dtype == BZ_F32) ? launch_general_kv<f16_t, float>(a, kv->kv_dtype, q_dtype, D, Gk, grid, s)
                                           : launch_general_kv<f16_t, f16_t>(a, kv->kv_dtype, q_dtype, D, Gk, grid, s);
            else
                rc = (out_dtype == BZ_F32) ? launch_general_kv<bf16_t, float>(a, kv->kv_dtype, q_dtype, D, Gk, grid, s)
                                           : launch_general_kv<bf16_t, bf16_t>(a, kv->kv_dtype, q_dtype, D, Gk, grid, s);
            if (rc == 0 && p->time_stop) BZ_CHECK_HIP(hipEventRecord(p->time_stop, s));
        }
        if (rc) return rc;
    }
    if (p->num_combos > 0) {
        if (out_dtype == BZ_F32) launch_combine<float>(p, bufs.part_o, bufs.part_lse, out, lse, num_qo_heads, D, s);
        else if (out_dtype == BZ_F16) launch_combine<f16_t>(p, bufs.part_o, bufs.part_lse, out, lse, num_qo_heads, D, s);
        else launch_combine<bf16_t>(p, bufs.part_o, bufs.part_lse, out, lse, num_qo_heads, D, s);
        BZ_LAUNCH_CHECK();
    }
    if (p->num_empty > 0) {
        const uint32_t row = num_qo_heads * D;
        if (out_dtype == BZ_F32) launch_zero<float>(p, out, row, s);
        else if (out_dtype == BZ_F16) launch_zero<f16_t>(p, out, row, s);
        else launch_zero<bf16_t>(p, out, row, s);
        BZ_LAUNCH_CHECK();
    }
    return 0;
}

} // namespace bz

using namespace bz;

// ------------------------------------------------------------------------------------------
// The library's own split-K scratch: a fixed device array that exists from module load to process
// exit, one copy per GPU.  Host code never passes the array's name to a kernel (on the host it is a
// stand-in, not a device address): the address is looked up once per device and kept.
// ------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char bz_decode_scratch[BZ_DECODE_NOALLOC_SCRATCH_BYTES];

namespace bz {

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {nullptr};

// Device address of this GPU's copy of the scratch array (looked up once per device, with that device
// current: by bz_decode_plan through decode_noalloc_prepare, so that bz_batch_decode_noalloc itself finds it
// there and does nothing but launch).
static int decode_scratch_for_current_device(unsigned char** ptr) {
    int dev = 0;
    BZ_CHECK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return BZ_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* sym = nullptr;
        BZ_CHECK_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(bz_decode_scratch)));
        if (!sym) return BZ_ERR_BAD_ARG;
        g_scratch_ptr[dev] = sym;
    }
    *ptr = static_cast<unsigned char*>(g_scratch_ptr[dev]);
    return 0;
}

int decode_noalloc_prepare() {
    unsigned char* ptr = nullptr;
    return decode_scratch_for_current_device(&ptr);
}

static inline size_t scratch_align(size_t x) { return (x + 255) / 256 * 256; }

} // namespace bz

extern "C" int bz_batch_decode(bz_decode_plan_t* plan_, const void* q, int q_dtype, const bz_paged_kv_t* kv,
                               void* out, int out_dtype, uint32_t num_qo_heads, int rope_mode, float rope_theta,
                               float sm_scale, const float* k_scale, const float* v_scale, float* lse,
                               void* stream) {
    return batch_decode_impl(reinterpret_cast<DecodePlan*>(plan_), q, q_dtype, kv, out, out_dtype, num_qo_heads,
                             rope_mode, rope_theta, sm_scale, k_scale, v_scale, lse, nullptr, stream);
}

extern "C" int bz_decode_step(bz_decode_plan_t* plan_, const void* q, int q_dtype, const void* k_new, const void* v_new,
                              const bz_paged_kv_t* kv, void* out, int out_dtype, uint32_t num_qo_heads, int rope,
                              float rope_theta, float sm_scale, const float* k_scale, const float* v_scale, float* lse,
                              void* stream) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p || !kv || !q || !k_new || !v_new || !out) return BZ_ERR_BAD_ARG;
    if (!p->planned) return BZ_ERR_NOT_PLANNED;
    if (!kv->k_data || !kv->v_data || !kv->indices || !kv->indptr || !kv->last_page_len) return BZ_ERR_BAD_ARG;
    if (kv->batch_size != p->batch_size || kv->page_size != p->page_size || kv->num_kv_heads != p->num_kv_heads ||
        kv->head_dim != p->head_dim || num_qo_heads != p->num_qo_heads)
        return BZ_ERR_BAD_ARG;
    if (q_dtype != BZ_F16 && q_dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED;
    if (out_dtype != q_dtype && out_dtype != BZ_F32) return BZ_ERR_UNSUPPORTED;
    if (kv->kv_dtype != q_dtype && kv->kv_dtype != BZ_E4M3) return BZ_ERR_UNSUPPORTED;
    hipStream_t s = (hipStream_t)stream;
    if (p->batch_size == 0) return 0;
    int rc = BZ_ERR_UNSUPPORTED;
    if (p->step_one_call && p->num_segments > 0) {
        const int D = (int)kv->head_dim;
        const float scale = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)D);
        const RopeFreqs freqs = make_rope_freqs(D, rope_theta > 0.f ? rope_theta : 1e4f);
        rc = decode_step_fast_path(p, q, k_new, v_new, out, lse, q_dtype, out_dtype, rope, scale * 1.4426950408889634f,
                                   freqs, kv, num_qo_heads, k_scale, v_scale, s);
        if (rc == 0 && p->num_empty > 0) { // sequences without pages: nothing to append, zero rows
            const uint32_t row = num_qo_heads * D;
            if (out_dtype == BZ_F32) launch_zero<float>(p, out, row, s);
            else if (out_dtype == BZ_F16) launch_zero<f16_t>(p, out, row, s);
            else launch_zero<bf16_t>(p, out, row, s);
            BZ_LAUNCH_CHECK();
        }
    }
    if (rc != BZ_ERR_UNSUPPORTED) return rc;
    // shapes the matrix-core kernel does not take, or a workspace without room for one partial per piece:
    // the same result from the two calls the step stands for
    rc = bz_append_decode_kv(kv, k_new, v_new, q_dtype, nullptr, 0, rope, rope_theta, k_scale, v_scale, stream);
    if (rc) return rc;
    return batch_decode_impl(p, q, q_dtype, kv, out, out_dtype, num_qo_heads, rope ? BZ_ROPE_Q_ONLY : BZ_ROPE_NONE,
                             rope_theta, sm_scale, k_scale, v_scale, lse, nullptr, stream);
}

extern "C" size_t bz_batch_decode_noalloc_scratch_bytes(void) { return BZ_DECODE_NOALLOC_SCRATCH_BYTES; }

extern "C" int bz_batch_decode_noalloc(bz_decode_plan_t* plan_, const void* q, int q_dtype, const bz_paged_kv_t* kv,
                                       void* out, int out_dtype, uint32_t num_qo_heads, int rope_mode,
                                       float rope_theta, float sm_scale, const float* k_scale, const float* v_scale,
                                       float* lse, void* stream) {
    DecodePlan* p = reinterpret_cast<DecodePlan*>(plan_);
    if (!p) return BZ_ERR_BAD_ARG;
    if (!p->planned) return BZ_ERR_NOT_PLANNED;
    // The partial results must fit the fixed array.  Which of the two kernels a call runs depends on its arguments
    // as well as on the plan, so the rule is the conservative one: what either kernel would need, unless the plan
    // is pinned to the general kernel.
    const size_t gen_o = scratch_align((size_t)p->num_partials * p->num_qo_heads * p->head_dim * sizeof(float));
    const size_t gen_l = scratch_align((size_t)p->num_partials * p->num_qo_heads * sizeof(float));
    const size_t mf_o = (p->mfma_ok && !p->force_general) ? scratch_align((size_t)p->mfma_partials * 16 * 128 * sizeof(float)) : 0;
    const size_t mf_l = (p->mfma_ok && !p->force_general) ? scratch_align((size_t)p->mfma_partials * 16 * sizeof(float)) : 0;
    if (gen_o + gen_l > (size_t)BZ_DECODE_NOALLOC_SCRATCH_BYTES || mf_o + mf_l > (size_t)BZ_DECODE_NOALLOC_SCRATCH_BYTES)
        return BZ_ERR_WORKSPACE;
    unsigned char* base = nullptr;
    const int rc = decode_scratch_for_current_device(&base);
    if (rc) return rc;
    // every partial row that the combine reads is written by the decode kernel of the same call first,
    // so nothing in the array has to start at zero
    const PartialBufs bufs = {reinterpret_cast<float*>(base), reinterpret_cast<float*>(base + gen_o),
                              reinterpret_cast<float*>(base), reinterpret_cast<float*>(base + mf_o)};
    return batch_decode_impl(p, q, q_dtype, kv, out, out_dtype, num_qo_heads, rope_mode, rope_theta, sm_scale, k_scale,
                             v_scale, lse, &bufs, stream);
}
