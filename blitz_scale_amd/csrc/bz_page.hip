// KV page writes for gfx950: prefill store and decode append, each optionally fused with the
// Llama rotate-half RoPE of the new K rows and of the matching q rows, and with e4m3
// quantisation for an fp8 pool.  Replaces src/kernel/page.cu of the BlitzScale worker; pool
// helpers replace the allocation at src/blitz/cache_manager.h:136-142 and the layer pointer
// bump at src/model/llama.h:378-381.
#include <cmath>

#include "bz_common.hpp"

namespace bz {

struct PageWriteArgs {
    char* k_data;
    char* v_data;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    const int32_t* steps_ahead; // optional: the table is this many decode steps ahead of the present
    const void* k_src;
    const void* v_src;
    void* q_inout;
    const int32_t* ragged_indptr; // prefill only
    const float* k_scale;
    const float* v_scale;
    uint64_t stride_page, stride_n, stride_h;
    uint32_t batch_size, page_size, num_kv_heads, num_qo_heads, num_tokens;
    int rope;
    RopeFreqs freqs;
};

// The rows of one token (q heads to rotate in place, then the k heads, then the v heads) on their way into
// page `page`, slot `slot` (page < 0: the token has no page; its rows are still rotated in place where the call
// rotates in place, and nothing goes to the pool).  A row of D elements is handled by D/16 lanes; each lane owns
// 8 elements of the lower half and the 8 elements of the upper half that form rotate-half pairs with them.
template <typename ST, typename PT, int D, bool PREFILL>
__device__ __forceinline__ void page_write_rows(const PageWriteArgs& a, int64_t page, int slot, size_t src_tok,
                                                const float* s_cos, const float* s_sin) {
    constexpr int LANES = D / 16;
    constexpr int ROWS = 256 / LANES;
    const int lane = threadIdx.x % LANES;
    // Pages written at prefill are next read by a later decode step, long after they have left the
    // caches: non-temporal stores leave the cache to the caller's q / k / v rows, which the attention
    // call reads next (16 prompts of 128..4096 tokens, 40 heads: 362 -> 353 us).
    auto pool_store = [](const Vec8<PT>& v, PT* p) {
        if (PREFILL) v.store_nt(p); else v.store(p);
    };
    const int Hq = (a.rope && a.q_inout) ? (int)a.num_qo_heads : 0;
    const int Hkv = (int)a.num_kv_heads;
    const int total_rows = Hq + 2 * Hkv;
    for (int r = threadIdx.x / LANES; r < total_rows; r += ROWS) {
        if (r < Hq) { // q row: rotate in place
            ST* row = reinterpret_cast<ST*>(a.q_inout) + (src_tok * a.num_qo_heads + r) * D;
            Vec8<ST> lo, hi;
            lo.load(row + lane * 8);
            hi.load(row + D / 2 + lane * 8);
            float x[8], y[8];
            lo.to_float(x);
            hi.to_float(y);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float c = s_cos[lane * 8 + e], s = s_sin[lane * 8 + e];
                float xr, yr;
                rope_pair(x[e], y[e], c, s, xr, yr);
                x[e] = xr;
                y[e] = yr;
            }
            lo.from_float(x);
            hi.from_float(y);
            lo.store(row + lane * 8);
            hi.store(row + D / 2 + lane * 8);
            continue;
        }
        const bool is_k = r < Hq + Hkv;
        const int h = is_k ? r - Hq : r - Hq - Hkv;
        const bool to_pool = page >= 0;
        const bool in_place = PREFILL && is_k && a.rope && (Hq > 0 || a.rope == 2);
        if (!to_pool && !in_place) continue;
        const ST* src = reinterpret_cast<const ST*>(is_k ? a.k_src : a.v_src) + (src_tok * Hkv + h) * D;
        char* pool = is_k ? a.k_data : a.v_data;
        const size_t off = ((size_t)page * a.stride_page + (size_t)slot * a.stride_n + (size_t)h * a.stride_h);
        PT* dst = reinterpret_cast<PT*>(pool) + off;
        Vec8<ST> lo, hi;
        lo.load(src + lane * 8);
        hi.load(src + D / 2 + lane * 8);
        const bool rotate = is_k && a.rope;
        const float* scale = is_k ? a.k_scale : a.v_scale;
        if constexpr (sizeof(ST) == sizeof(PT)) {
            if (!rotate && !scale) { // bit-exact copy
                Vec8<PT> l2, h2;
                l2.raw = lo.raw;
                h2.raw = hi.raw;
                pool_store(l2, dst + lane * 8);
                pool_store(h2, dst + D / 2 + lane * 8);
                continue;
            }
        }
        float x[8], y[8];
        lo.to_float(x);
        hi.to_float(y);
        if (rotate) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float c = s_cos[lane * 8 + e], s = s_sin[lane * 8 + e];
                float xr, yr;
                rope_pair(x[e], y[e], c, s, xr, yr);
                x[e] = xr;
                y[e] = yr;
            }
        }
        if (PREFILL && rotate && (Hq > 0 || a.rope == 2)) {
            // fused RoPE of the prefill path: the caller's k rows are rotated in place as well, so the
            // attention call that follows contracts rotated q with rotated k
            Vec8<ST> lr, hr;
            lr.from_float(x);
            hr.from_float(y);
            ST* srcw = const_cast<ST*>(src);
            lr.store(srcw + lane * 8);
            hr.store(srcw + D / 2 + lane * 8);
        }
        if (!to_pool) continue;
        if (scale) {
            const float sc = scale[h];
#pragma unroll
            for (int e = 0; e < 8; ++e) { x[e] = x[e] / sc; y[e] = y[e] / sc; }
        }
        Vec8<PT> l2, h2;
        l2.from_float(x);
        h2.from_float(y);
        pool_store(l2, dst + lane * 8);
        pool_store(h2, dst + D / 2 + lane * 8);
    }
}

template <typename ST, typename PT, int D, bool PREFILL>
__global__ __launch_bounds__(256) void page_write_kernel(PageWriteArgs a) {
    __shared__ float s_cos[D / 2], s_sin[D / 2];

    // Prefill: one token per workgroup and pass.  The launch has one workgroup per token when the host
    // knows the token count, otherwise a fixed number of workgroups that stride over the tokens counted
    // by the ragged index itself (ragged_indptr[batch_size], read on the device).
    const int total = PREFILL ? (int)min((uint32_t)max(a.ragged_indptr[a.batch_size], 0), a.num_tokens) : (int)a.batch_size;
    for (int unit = blockIdx.x; unit < total; unit += gridDim.x) {
        int b, pos;
        size_t src_tok;
        bool no_page = false;
        if (PREFILL) {
            const int n = unit; // global token index; largest b with ragged_indptr[b] <= n (wave-uniform search)
            int lo = 0, hi = (int)a.batch_size;
            while (hi - lo > 1) {
                const int mid = (lo + hi) / 2;
                if (a.ragged_indptr[mid] <= n) lo = mid; else hi = mid;
            }
            b = lo;
            pos = n - a.ragged_indptr[b];
            src_tok = (size_t)n;
            // a request longer than the pages its table row lists (the reference asserts seq_len >= append
            // length, src/kernel/page.cu:43): the tokens without a page are not cached -- nothing is written
            // outside the listed pages -- but a call that rotates q / k in place still rotates their rows, so
            // that the attention call which follows sees every row of the request rotated alike
            no_page = pos / (int)a.page_size >= a.indptr[b + 1] - a.indptr[b];
            if (no_page && !(a.rope && (a.q_inout || a.rope == 2))) continue;
        } else {
            b = unit;
            const int ahead = a.steps_ahead ? *a.steps_ahead : 0; // fetched together with the table entries
            const int np = a.indptr[b + 1] - a.indptr[b];
            if (np <= 0) continue;
            pos = (np - 1) * (int)a.page_size + a.last_page_len[b] - 1 - max(ahead, 0);
            if (pos < 0) continue; // the sequence has no token yet at the present step
            src_tok = (size_t)b;
        }
        const int64_t page = no_page ? -1 : a.indices[a.indptr[b] + pos / (int)a.page_size];
        const int slot = pos % (int)a.page_size;

        if (a.rope) {
            __syncthreads(); // the previous pass has finished with the table
            for (int i = threadIdx.x; i < D / 2; i += 256) {
                float s, c;
                sincosf((float)pos * a.freqs.f[i], &s, &c);
                s_cos[i] = c;
                s_sin[i] = s;
            }
            __syncthreads();
        }
        page_write_rows<ST, PT, D, PREFILL>(a, page, slot, src_tok, s_cos, s_sin);
    }
}

// Decode append: one workgroup per sequence, one new row per (q | k | v) head.  At decode batch sizes the
// kernel is nothing but its chain of dependent memory round trips, so everything that does not depend
// on the page table (the counter, the table entries themselves, the caller's q / k / v rows) is
// requested up front; the page id is the one dependent fetch and overlaps with the angles.
template <typename ST, typename PT, int D>
__global__ __launch_bounds__(256) void append_kernel(PageWriteArgs a) {
    constexpr int LANES = D / 16;
    constexpr int ROWS = 256 / LANES;
    constexpr int MAXR = 4; // rows per lane group held in registers; more rows take the loop at the end
    __shared__ float s_cos[D / 2], s_sin[D / 2];

    const int b = blockIdx.x;
    const int ahead = a.steps_ahead ? *a.steps_ahead : 0;
    const int ip0 = a.indptr[b], ip1 = a.indptr[b + 1];
    const int lpl = a.last_page_len[b];
    const int lane = threadIdx.x % LANES, r0 = threadIdx.x / LANES;
    const int Hq = (a.rope && a.q_inout) ? (int)a.num_qo_heads : 0;
    const int Hkv = (int)a.num_kv_heads;
    const int total_rows = Hq + 2 * Hkv;
    auto row_src = [&](int r) -> const ST* { // rows 0..Hq-1: q heads, then the k heads, then the v heads
        if (r < Hq) return reinterpret_cast<const ST*>(a.q_inout) + ((size_t)b * a.num_qo_heads + r) * D;
        const bool is_k = r < Hq + Hkv;
        return reinterpret_cast<const ST*>(is_k ? a.k_src : a.v_src) + ((size_t)b * Hkv + (is_k ? r - Hq : r - Hq - Hkv)) * D;
    };
    Vec8<ST> lo[MAXR], hi[MAXR];
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
        const int r = r0 + i * ROWS;
        if (r < total_rows) {
            const ST* src = row_src(r);
            lo[i].load(src + lane * 8);
            hi[i].load(src + D / 2 + lane * 8);
        }
    }
    const int np = ip1 - ip0;
    if (np <= 0) return;
    const int pos = (np - 1) * (int)a.page_size + lpl - 1 - max(ahead, 0);
    if (pos < 0) return; // the sequence has no token yet at the present step
    const int64_t page = a.indices[ip0 + pos / (int)a.page_size];
    const int slot = pos % (int)a.page_size;
    if (a.rope) {
        for (int i = threadIdx.x; i < D / 2; i += 256) {
            float s, c;
            sincosf((float)pos * a.freqs.f[i], &s, &c);
            s_cos[i] = c;
            s_sin[i] = s;
        }
        __syncthreads();
    }
    auto finish_row = [&](int r, Vec8<ST>& l, Vec8<ST>& h) {
        const bool is_q = r < Hq, is_k = !is_q && r < Hq + Hkv;
        const bool rotate = (is_q || is_k) && a.rope;
        float x[8], y[8];
        if (is_q || rotate || (is_k ? a.k_scale : a.v_scale) || sizeof(ST) != sizeof(PT)) {
            l.to_float(x);
            h.to_float(y);
        }
        if (rotate) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float c = s_cos[lane * 8 + e], sn = s_sin[lane * 8 + e];
                float xr, yr;
                rope_pair(x[e], y[e], c, sn, xr, yr);
                x[e] = xr;
                y[e] = yr;
            }
        }
        if (is_q) { // rotated in place
            ST* row = const_cast<ST*>(row_src(r));
            l.from_float(x);
            h.from_float(y);
            l.store(row + lane * 8);
            h.store(row + D / 2 + lane * 8);
            return;
        }
        const int hd = is_k ? r - Hq : r - Hq - Hkv;
        PT* dst = reinterpret_cast<PT*>(is_k ? a.k_data : a.v_data) +
                  ((size_t)page * a.stride_page + (size_t)slot * a.stride_n + (size_t)hd * a.stride_h);
        const float* scale = is_k ? a.k_scale : a.v_scale;
        Vec8<PT> l2, h2;
        if constexpr (sizeof(ST) == sizeof(PT)) {
            if (!rotate && !scale) { // bit-exact copy
                l2.raw = l.raw;
                h2.raw = h.raw;
                l2.store(dst + lane * 8);
                h2.store(dst + D / 2 + lane * 8);
                return;
            }
        }
        if (scale) {
            const float sc = scale[hd];
#pragma unroll
            for (int e = 0; e < 8; ++e) { x[e] = x[e] / sc; y[e] = y[e] / sc; }
        }
        l2.from_float(x);
        h2.from_float(y);
        l2.store(dst + lane * 8);
        h2.store(dst + D / 2 + lane * 8);
    };
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
        const int r = r0 + i * ROWS;
        if (r < total_rows) finish_row(r, lo[i], hi[i]);
    }
    for (int r = r0 + MAXR * ROWS; r < total_rows; r += ROWS) {
        Vec8<ST> l, h;
        const ST* src = row_src(r);
        l.load(src + lane * 8);
        h.load(src + D / 2 + lane * 8);
        finish_row(r, l, h);
    }
}

template <typename ST, typename PT, bool PREFILL>
static int launch_page_write_d(const PageWriteArgs& a, int D, uint32_t grid, hipStream_t s) {
    if (grid == 0) return 0;
    if constexpr (PREFILL) {
        if (D == 128) hipLaunchKernelGGL((page_write_kernel<ST, PT, 128, true>), dim3(grid), dim3(256), 0, s, a);
        else if (D == 64) hipLaunchKernelGGL((page_write_kernel<ST, PT, 64, true>), dim3(grid), dim3(256), 0, s, a);
        else return BZ_ERR_UNSUPPORTED;
    } else {
        if (D == 128) hipLaunchKernelGGL((append_kernel<ST, PT, 128>), dim3(grid), dim3(256), 0, s, a);
        else if (D == 64) hipLaunchKernelGGL((append_kernel<ST, PT, 64>), dim3(grid), dim3(256), 0, s, a);
        else return BZ_ERR_UNSUPPORTED;
    }
    BZ_LAUNCH_CHECK();
    return 0;
}

template <bool PREFILL>
static int launch_page_write(const PageWriteArgs& a, int src_dtype, int pool_dtype, int D, uint32_t grid,
                             hipStream_t s) {
    if (src_dtype == BZ_F16 && pool_dtype == BZ_F16) return launch_page_write_d<f16_t, f16_t, PREFILL>(a, D, grid, s);
    if (src_dtype == BZ_BF16 && pool_dtype == BZ_BF16) return launch_page_write_d<bf16_t, bf16_t, PREFILL>(a, D, grid, s);
    if (src_dtype == BZ_F16 && pool_dtype == BZ_E4M3) return launch_page_write_d<f16_t, e4m3_t, PREFILL>(a, D, grid, s);
    if (src_dtype == BZ_BF16 && pool_dtype == BZ_E4M3) return launch_page_write_d<bf16_t, e4m3_t, PREFILL>(a, D, grid, s);
    return BZ_ERR_UNSUPPORTED;
}

static int fill_args(PageWriteArgs& a, const bz_paged_kv_t* kv, const void* k, const void* v, void* q_inout,
                     uint32_t num_qo_heads, int rope, float rope_theta, const float* k_scale, const float* v_scale,
                     bool prefill) {
    if (!kv || !k || !v || !kv->k_data || !kv->v_data) return BZ_ERR_BAD_ARG;
    if (!kv->indices || !kv->indptr || (!prefill && !kv->last_page_len)) return BZ_ERR_BAD_ARG;
    if (kv->stride_n % 8 || kv->stride_h % 8 || kv->stride_page % 8) return BZ_ERR_BAD_ARG;
    a.k_data = (char*)kv->k_data; a.v_data = (char*)kv->v_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.steps_ahead = kv->steps_ahead;
    a.k_src = k; a.v_src = v; a.q_inout = q_inout; a.ragged_indptr = nullptr;
    a.k_scale = k_scale; a.v_scale = v_scale;
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.batch_size = kv->batch_size; a.page_size = kv->page_size; a.num_kv_heads = kv->num_kv_heads;
    a.num_qo_heads = num_qo_heads; a.num_tokens = 0;
    a.rope = rope == 2 ? 2 : (rope ? 1 : 0);
    a.freqs = make_rope_freqs((int)kv->head_dim, rope_theta > 0.f ? rope_theta : 1e4f);
    return 0;
}

// ---- one pass over the cached K rows of a page table: rotate them in place at their positions (direction +1) or
// take the rotation off again (direction -1).  A cache that arrives with K as the projection left it -- the
// reference's convention, whose decode call rotates every cached row at every step (attention_decode.cu:35) -- is
// brought to this library's convention (K cached rotated, the decode kernels rotate q only) once, at the speed of
// a copy, instead of paying for the rotation at every step; a cache that leaves for such a consumer is taken back.
// Workgroup (b, c) takes pages c, c + gridDim.y, ... of sequence b: the angles of a page's slots go through LDS
// (they are shared by the kv heads), eight lanes per row as in the page writes.
struct RopeCachedArgs {
    char* k_data;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    uint64_t stride_page, stride_n, stride_h;
    uint32_t page_size, num_kv_heads;
    float direction;
    RopeFreqs freqs;
};

template <typename PT, int D>
__global__ __launch_bounds__(256) void rope_cached_k_kernel(RopeCachedArgs a) {
    extern __shared__ float2 s_cs[]; // [slot][pair]
    constexpr int LANES = D / 16;
    const int b = blockIdx.x;
    const int ip0 = a.indptr[b], np = a.indptr[b + 1] - ip0;
    if (np <= 0) return;
    const int P = (int)a.page_size, Hkv = (int)a.num_kv_heads;
    const int lane = threadIdx.x % LANES;
    for (int pg = blockIdx.y; pg < np; pg += gridDim.y) {
        const int slots = pg + 1 < np ? P : min(max(a.last_page_len[b], 0), P);
        const int64_t page = a.indices[ip0 + pg];
        __syncthreads(); // the previous page's angles are no longer read
        for (int i = threadIdx.x; i < slots * (D / 2); i += 256) {
            float sn, cs;
            sincosf((float)(pg * P + i / (D / 2)) * a.freqs.f[i % (D / 2)], &sn, &cs);
            s_cs[i] = make_float2(cs, a.direction * sn);
        }
        __syncthreads();
        for (int r = threadIdx.x / LANES; r < slots * Hkv; r += 256 / LANES) {
            const int slot = r / Hkv, h = r % Hkv;
            PT* row = reinterpret_cast<PT*>(a.k_data) +
                      ((size_t)page * a.stride_page + (size_t)slot * a.stride_n + (size_t)h * a.stride_h);
            Vec8<PT> lo, hi;
            lo.load(row + lane * 8);
            hi.load(row + D / 2 + lane * 8);
            float x[8], y[8];
            lo.to_float(x);
            hi.to_float(y);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float2 cs = s_cs[slot * (D / 2) + lane * 8 + e];
                float xr, yr;
                rope_pair(x[e], y[e], cs.x, cs.y, xr, yr);
                x[e] = xr;
                y[e] = yr;
            }
            lo.from_float(x);
            hi.from_float(y);
            lo.store(row + lane * 8);
            hi.store(row + D / 2 + lane * 8);
        }
    }
}

__global__ void steps_ahead_advance_kernel(int32_t* steps_ahead) {
    const int32_t v = *steps_ahead;
    if (v > 0) *steps_ahead = v - 1;
}

} // namespace bz

using namespace bz;

extern "C" int bz_steps_ahead_advance(int32_t* steps_ahead, void* stream) {
    if (!steps_ahead) return BZ_ERR_BAD_ARG;
    hipLaunchKernelGGL(steps_ahead_advance_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, steps_ahead);
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_store_prefill_kv(const bz_paged_kv_t* kv, void* k, const void* v, int src_dtype,
                                   const int32_t* ragged_indptr, uint32_t num_tokens, void* q_inout,
                                   uint32_t num_qo_heads, int rope, float rope_theta, const float* k_scale,
                                   const float* v_scale, void* stream) {
    PageWriteArgs a;
    int rc = fill_args(a, kv, k, v, q_inout, num_qo_heads, rope, rope_theta, k_scale, v_scale, true);
    if (rc) return rc;
    if (!ragged_indptr) return BZ_ERR_BAD_ARG;
    a.ragged_indptr = ragged_indptr;
    a.num_tokens = num_tokens;
    if (kv->batch_size == 0) return 0;
    // One workgroup per token when the caller knows the count; otherwise (the reference's four-argument
    // call, src/kernel/page.h:66-67, whose launch is shaped by page size and batch alone, page.cu:84-89) a
    // fixed launch whose workgroups stride over the tokens that ragged_indptr[batch_size] counts.
    const uint32_t grid = num_tokens == BZ_NUM_TOKENS_FROM_INDPTR ? 8192u : num_tokens;
    return launch_page_write<true>(a, src_dtype, kv->kv_dtype, (int)kv->head_dim, grid, (hipStream_t)stream);
}

extern "C" int bz_append_decode_kv(const bz_paged_kv_t* kv, const void* k, const void* v, int src_dtype,
                                   void* q_inout, uint32_t num_qo_heads, int rope, float rope_theta,
                                   const float* k_scale, const float* v_scale, void* stream) {
    PageWriteArgs a;
    int rc = fill_args(a, kv, k, v, q_inout, num_qo_heads, rope, rope_theta, k_scale, v_scale, false);
    if (rc) return rc;
    return launch_page_write<false>(a, src_dtype, kv->kv_dtype, (int)kv->head_dim, kv->batch_size,
                                    (hipStream_t)stream);
}

extern "C" int bz_rope_cached_k(const bz_paged_kv_t* kv, float rope_theta, int inverse, void* stream) {
    if (!kv || !kv->k_data || !kv->indices || !kv->indptr || !kv->last_page_len) return BZ_ERR_BAD_ARG;
    if (kv->stride_n % 8 || kv->stride_h % 8 || kv->stride_page % 8 || kv->page_size == 0) return BZ_ERR_BAD_ARG;
    if (kv->kv_dtype != BZ_F16 && kv->kv_dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED; // (e4m3 rows would be requantised)
    const int D = (int)kv->head_dim;
    if (D != 128 && D != 64) return BZ_ERR_UNSUPPORTED;
    const size_t lds = (size_t)kv->page_size * (D / 2) * sizeof(float2);
    if (lds > 64 * 1024) return BZ_ERR_UNSUPPORTED; // page_size <= 128 (head_dim 128) / 256 (head_dim 64)
    if (kv->batch_size == 0) return 0;
    RopeCachedArgs a;
    a.k_data = (char*)kv->k_data;
    a.indices = kv->indices; a.indptr = kv->indptr; a.last_page_len = kv->last_page_len;
    a.stride_page = kv->stride_page; a.stride_n = kv->stride_n; a.stride_h = kv->stride_h;
    a.page_size = kv->page_size; a.num_kv_heads = kv->num_kv_heads;
    a.direction = inverse ? -1.0f : 1.0f;
    a.freqs = make_rope_freqs(D, rope_theta > 0.f ? rope_theta : 1e4f);
    const dim3 grid(kv->batch_size, 32);
    hipStream_t s = (hipStream_t)stream;
    if (kv->kv_dtype == BZ_F16) {
        if (D == 128) hipLaunchKernelGGL((rope_cached_k_kernel<f16_t, 128>), grid, dim3(256), lds, s, a);
        else hipLaunchKernelGGL((rope_cached_k_kernel<f16_t, 64>), grid, dim3(256), lds, s, a);
    } else {
        if (D == 128) hipLaunchKernelGGL((rope_cached_k_kernel<bf16_t, 128>), grid, dim3(256), lds, s, a);
        else hipLaunchKernelGGL((rope_cached_k_kernel<bf16_t, 64>), grid, dim3(256), lds, s, a);
    }
    BZ_LAUNCH_CHECK();
    return 0;
}

// ---- pool helpers -----------------------------------------------------------------------------
extern "C" void bz_paged_kv_set_layout(bz_paged_kv_t* kv, int layout) {
    const uint64_t H = kv->num_kv_heads, P = kv->page_size, D = kv->head_dim;
    kv->stride_page = 2 * H * P * D;
    if (layout == BZ_LAYOUT_HND) { kv->stride_n = D; kv->stride_h = P * D; }
    else { kv->stride_n = H * D; kv->stride_h = D; }
}

extern "C" uint64_t bz_kv_pool_bytes(uint32_t num_layers, uint64_t max_pages, uint32_t num_kv_heads,
                                     uint32_t page_size, uint32_t head_dim, int kv_dtype) {
    return (uint64_t)2 * num_layers * max_pages * num_kv_heads * page_size * head_dim * dtype_bytes(kv_dtype);
}

extern "C" int bz_kv_pool_alloc(void** base, uint64_t bytes) {
    if (!base) return BZ_ERR_BAD_ARG;
    return (int)hipMalloc(base, (size_t)bytes);
}

extern "C" int bz_kv_pool_free(void* base) { return (int)hipFree(base); }

extern "C" void bz_kv_layer_view(bz_paged_kv_t* kv, void* pool_base, uint32_t layer, uint64_t max_pages) {
    const uint64_t es = dtype_bytes(kv->kv_dtype);
    char* k = (char*)pool_base + (uint64_t)layer * max_pages * kv->stride_page * es;
    kv->k_data = k;
    kv->v_data = k + (kv->stride_page / 2) * es;
}

extern "C" const char* bz_build_info(void) { return "blitz-scale paged-attention path, gfx950, wave64"; }

extern "C" const char* bz_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case BZ_ERR_BAD_ARG: return "bz: invalid argument";
        case BZ_ERR_UNSUPPORTED: return "bz: unsupported shape or type";
        case BZ_ERR_WORKSPACE: return "bz: workspace too small";
        case BZ_ERR_NOT_PLANNED: return "bz: plan() has not been called";
        case BZ_ERR_NO_PAGES: return "bz: out of KV pages";
        default: return hipGetErrorString((hipError_t)code);
    }
}
