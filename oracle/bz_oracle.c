/*
 * bz_oracle.c -- TEST INFRASTRUCTURE ONLY.  Scalar, fp32-accumulate CPU
 * restatement of the paged-attention compute path of the BlitzScale C++
 * worker.  It is the checker the HIP kernels are compared with; nothing in the
 * shipped library links, loads or calls it.
 *
 * What each function follows (paths relative to the reference checkout):
 *   page addressing / strides ........ src/kernel/page.h:12-64
 *   sequence length formula .......... src/kernel/page.cu:38-40
 *   prefill store placement .......... src/kernel/page.cu:21-62
 *   decode append placement .......... src/kernel/page.cu:96-115 (position
 *                                      seq_len-1: last page, slot last_page_len-1)
 *   batch decode call semantics ...... src/kernel/attention_decode.cu:13-40
 *   ragged causal prefill semantics .. src/kernel/attention_prefill.cu:11-46
 *   rms_norm / add_rms_norm .......... src/kernel/rms_norm.h:11-34, norm.cu:7-39
 *   silu_and_mul ..................... src/kernel/activation.h:7-16, activation.cu:9
 *   add_residual ..................... src/kernel/add.h:8-14, add.cu:13-38
 *   embedding ........................ src/kernel/embedding.h:7-36, embedding.cu:7-47
 *   gather_last_token / batch_find_max src/kernel/sampler.h:8-26, sampler.cu:7-25,80-109
 *   host page table build / grow ..... src/blitz/batch.h:236-257,
 *                                      src/blitz/cache_manager.h:161-184,197-324
 *   row-major (batched) GEMM ......... src/util/cublas_wrapper.h:33-88,144-207
 *
 * The arithmetic behind the attention / norm / activation calls lives in a
 * FlashInfer fork that is absent from the reference checkout
 * (.gitmodules:1-4, src/kernel/flashinfer/ empty), so these functions restate
 * the published algorithm (softmax(s q k^T) v with s = 1/sqrt(D), Llama
 * rotate-half RoPE, x * rsqrt(mean(x^2)+eps) * w, x/(1+exp(-x)) * y) and are
 * pinned by closed forms, invariants and an independent float64 dense
 * implementation in tests/ rather than by reference fixtures (the reference has
 * none for this path).
 *
 * Storage types are passed as raw bits: f16 / bf16 as uint16_t, e4m3 (OCP
 * e4m3fn, max 448, no inf) as uint8_t.  All accumulation is fp32, sequential.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define BZO_F16 0
#define BZO_BF16 1
#define BZO_E4M3 2
#define BZO_F32 3

#define BZO_ROPE_NONE 0
#define BZO_ROPE_Q_ONLY 1 /* rotate q at seq_len-1; cached K already rotated */
#define BZO_ROPE_FULL 2   /* rotate q at seq_len-1 and every cached K at its position */

/* ------------------------------------------------------------------ */
/* scalar conversions                                                  */
/* ------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float bzo_f16_to_f32(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0) {
        if (m == 0) return u2f(s);
        /* subnormal: value = m * 2^-24 */
        float v = (float)m * (1.0f / 16777216.0f);
        return (s ? -v : v);
    }
    if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
    return u2f(s | ((e + 112u) << 23) | (m << 13));
}

uint16_t bzo_f32_to_f16(float f) { /* round-to-nearest-even */
    uint32_t u = f2u(f);
    uint16_t s = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint16_t)(s | 0x7c00u | ((a > 0x7f800000u) ? 0x200u : 0));
    if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);           /* rounds to inf: >= 65520 */
    if (a < 0x33000001u) return s;                                   /* <= 2^-25: rounds to zero */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7fffffu) | 0x800000u;                        /* 24-bit significand */
    int shift;                                                       /* bits dropped */
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }
    else         { shift = 13;             base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }
    uint32_t q = m >> shift, r = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (r > half || (r == half && (q & 1u))) q++;
    return (uint16_t)(s | (base + q));                               /* carry propagates into exponent */
}

float bzo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t bzo_f32_to_bf16(float f) { /* round-to-nearest-even */
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    uint32_t r = 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)((u + r) >> 16);
}

/* OCP e4m3fn: 1-4-3, bias 7, no infinity, S.1111.111 is NaN, max finite 448 */
float bzo_e4m3_to_f32(uint8_t b) {
    int s = b >> 7, e = (b >> 3) & 0xf, m = b & 7;
    float v;
    if (e == 15 && m == 7) return u2f(0x7fc00000u);
    if (e == 0) v = ldexpf((float)m, -9);           /* m/8 * 2^-6 */
    else        v = ldexpf((float)(8 + m), e - 10); /* (1+m/8) * 2^(e-7) */
    return s ? -v : v;
}

uint8_t bzo_f32_to_e4m3(float f) { /* RNE, saturating to +-448, NaN -> 0x7f */
    if (f != f) return 0x7f;
    uint8_t s = (f2u(f) >> 31) ? 0x80 : 0;
    float a = fabsf(f);
    if (a >= 448.0f) return (uint8_t)(s | 0x7e);
    /* nearest-even over the 127 non-negative finite codes, by bisection */
    int lo = 0, hi = 0x7e;
    while (hi - lo > 1) {
        int mid = (lo + hi) / 2;
        if (bzo_e4m3_to_f32((uint8_t)mid) <= a) lo = mid; else hi = mid;
    }
    float vlo = bzo_e4m3_to_f32((uint8_t)lo), vhi = bzo_e4m3_to_f32((uint8_t)hi);
    float dlo = a - vlo, dhi = vhi - a; /* both exact in fp32: few significant bits apart */
    int pick;
    if (dlo < dhi) pick = lo; else if (dhi < dlo) pick = hi; else pick = (lo & 1) ? hi : lo;
    return (uint8_t)(s | pick);
}

static inline float load_as_f32(const void* p, int dtype, size_t i) {
    switch (dtype) {
        case BZO_F16:  return bzo_f16_to_f32(((const uint16_t*)p)[i]);
        case BZO_BF16: return bzo_bf16_to_f32(((const uint16_t*)p)[i]);
        case BZO_E4M3: return bzo_e4m3_to_f32(((const uint8_t*)p)[i]);
        default:       return ((const float*)p)[i];
    }
}
static inline void store_from_f32(void* p, int dtype, size_t i, float v) {
    switch (dtype) {
        case BZO_F16:  ((uint16_t*)p)[i] = bzo_f32_to_f16(v); break;
        case BZO_BF16: ((uint16_t*)p)[i] = bzo_f32_to_bf16(v); break;
        case BZO_E4M3: ((uint8_t*)p)[i] = bzo_f32_to_e4m3(v); break;
        default:       ((float*)p)[i] = v; break;
    }
}
static inline size_t dtype_size(int dtype) {
    return dtype == BZO_F32 ? 4 : (dtype == BZO_E4M3 ? 1 : 2);
}

void bzo_to_f32(const void* src, int dtype, size_t n, float* dst) {
    for (size_t i = 0; i < n; ++i) dst[i] = load_as_f32(src, dtype, i);
}
void bzo_from_f32(const float* src, int dtype, size_t n, void* dst) {
    for (size_t i = 0; i < n; ++i) store_from_f32(dst, dtype, i, src[i]);
}

/* ------------------------------------------------------------------ */
/* RoPE: Llama rotate-half.  For i < D/2 with f_i = theta^(-2i/D):      */
/*   x_i'       = x_i cos(p f_i) - x_{i+D/2} sin(p f_i)                 */
/*   x_{i+D/2}' = x_{i+D/2} cos(p f_i) + x_i sin(p f_i)                 */
/* f_i is evaluated in double and rounded to fp32; the angle p*f_i is   */
/* one fp32 multiply; sin/cos are the correctly rounded values of that  */
/* fp32 angle.  (No reference function exists: RoPE is only the         */
/* kRoPELlama flag at attention_decode.cu:35 / attention_prefill.cu:38.)*/
/* ------------------------------------------------------------------ */
void bzo_rope_freqs(int D, float theta, float* freq /* [D/2] */) {
    for (int i = 0; i < D / 2; ++i)
        freq[i] = (float)pow((double)theta, -2.0 * (double)i / (double)D);
}

void bzo_rope_llama(float* x, int D, int pos, float theta) {
    int half = D / 2;
    for (int i = 0; i < half; ++i) {
        float f = (float)pow((double)theta, -2.0 * (double)i / (double)D);
        float ang = (float)pos * f;
        float c = (float)cos((double)ang), s = (float)sin((double)ang);
        float a = x[i], b = x[i + half];
        x[i] = a * c - b * s;
        x[i + half] = b * c + a * s;
    }
}

/* rotate rows of a ragged [N, H, D] tensor in place by position inside the request,
 * rounding back to the storage dtype */
void bzo_rope_ragged_inplace(void* x, int dtype, const int32_t* indptr, int B, int H, int D, float theta) {
    float* row = (float*)malloc(sizeof(float) * (size_t)D);
    for (int b = 0; b < B; ++b)
        for (int t = indptr[b]; t < indptr[b + 1]; ++t)
            for (int h = 0; h < H; ++h) {
                size_t off = ((size_t)t * H + h) * D;
                for (int d = 0; d < D; ++d) row[d] = load_as_f32(x, dtype, off + d);
                bzo_rope_llama(row, D, t - indptr[b], theta);
                for (int d = 0; d < D; ++d) store_from_f32(x, dtype, off + d, row[d]);
            }
    free(row);
}

/* ------------------------------------------------------------------ */
/* paged KV: description of one layer plane of the pool                 */
/* element address = page*stride_page + slot*stride_n + head*stride_h + d
 * relative to k_base / v_base (page.h:24-32,42-43)                     */
/* ------------------------------------------------------------------ */
typedef struct {
    const void* k_base;
    const void* v_base;
    const int32_t* indices;
    const int32_t* indptr;
    const int32_t* last_page_len;
    int32_t batch_size, page_size, num_kv_heads, head_dim;
    int64_t stride_page, stride_n, stride_h; /* in elements */
    int32_t kv_dtype;
} bzo_paged_kv;

static inline int64_t seq_len_of(const bzo_paged_kv* kv, int b) {
    int32_t np = kv->indptr[b + 1] - kv->indptr[b];
    if (np <= 0) return 0;
    return (int64_t)(np - 1) * kv->page_size + kv->last_page_len[b]; /* page.cu:38-40 */
}

void bzo_seq_lens(const bzo_paged_kv* kv, int64_t* out) {
    for (int b = 0; b < kv->batch_size; ++b) out[b] = seq_len_of(kv, b);
}

static inline int64_t kv_elem_off(const bzo_paged_kv* kv, int b, int64_t j, int head) {
    int64_t page = kv->indices[kv->indptr[b] + j / kv->page_size];
    int64_t slot = j % kv->page_size;
    return page * kv->stride_page + slot * kv->stride_n + (int64_t)head * kv->stride_h;
}

/* ------------------------------------------------------------------ */
/* batch decode: o[b,h,:] = sum_j softmax_j(s q.k_j) v_j, j < seq_len_b */
/* g(h) = h / (Hq/Hkv).  k_scale / v_scale: optional per-kv-head fp32   */
/* dequantisation factors (NULL = 1).  out is fp32 [B,Hq,D].            */
/* lse (optional, [B,Hq]) = m + log(l) of the scaled logits.            */
/* ------------------------------------------------------------------ */
void bzo_batch_decode(const void* q, int q_dtype, const bzo_paged_kv* kv, int num_qo_heads,
                      int rope_mode, float rope_theta, float sm_scale,
                      const float* k_scale, const float* v_scale, float* out, float* lse) {
    const int D = kv->head_dim, Hq = num_qo_heads, Hkv = kv->num_kv_heads, G = Hq / Hkv;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1)
#endif
    for (int b = 0; b < kv->batch_size; ++b) {
        int64_t L = seq_len_of(kv, b);
        float* s = (float*)malloc(sizeof(float) * (size_t)(L > 0 ? L : 1));
        float* qv = (float*)malloc(sizeof(float) * D);
        float* kr = (float*)malloc(sizeof(float) * D);
        for (int h = 0; h < Hq; ++h) {
            int kvh = h / G;
            float* o = out + ((size_t)b * Hq + h) * D;
            for (int d = 0; d < D; ++d) o[d] = 0.0f;
            if (L == 0) { if (lse) lse[(size_t)b * Hq + h] = -INFINITY; continue; }
            for (int d = 0; d < D; ++d) qv[d] = load_as_f32(q, q_dtype, ((size_t)b * Hq + h) * D + d);
            if (rope_mode != BZO_ROPE_NONE) bzo_rope_llama(qv, D, (int)(L - 1), rope_theta);
            float ks = k_scale ? k_scale[kvh] : 1.0f, vs = v_scale ? v_scale[kvh] : 1.0f;
            float m = -INFINITY;
            for (int64_t j = 0; j < L; ++j) {
                int64_t off = kv_elem_off(kv, b, j, kvh);
                for (int d = 0; d < D; ++d) kr[d] = load_as_f32(kv->k_base, kv->kv_dtype, (size_t)(off + d));
                if (rope_mode == BZO_ROPE_FULL) bzo_rope_llama(kr, D, (int)j, rope_theta);
                float acc = 0.0f;
                for (int d = 0; d < D; ++d) acc += qv[d] * kr[d];
                s[j] = acc * ks * sm_scale;
                if (s[j] > m) m = s[j];
            }
            float l = 0.0f;
            for (int64_t j = 0; j < L; ++j) {
                float p = expf(s[j] - m);
                l += p;
                int64_t off = kv_elem_off(kv, b, j, kvh);
                for (int d = 0; d < D; ++d)
                    o[d] += p * load_as_f32(kv->v_base, kv->kv_dtype, (size_t)(off + d));
            }
            float inv = vs / l;
            for (int d = 0; d < D; ++d) o[d] *= inv;
            if (lse) lse[(size_t)b * Hq + h] = m + logf(l);
        }
        free(s); free(qv); free(kr);
    }
}

/* ------------------------------------------------------------------ */
/* ragged causal prefill self-attention (attention_prefill.cu:26-40):   */
/* q [N,Hq,D], k,v [N,Hkv,D], indptr [B+1] used for both q and kv.      */
/* Token i of request r attends to tokens j<=i of r (causal != 0) or to */
/* every token of r (causal == 0).  rope != 0: q and k are rotated by   */
/* their offset inside the request before the dot product (fp32, not    */
/* rounded back).  rows: optional list of n_rows global token ids to    */
/* evaluate (NULL = all); out is fp32 [n_rows or N, Hq, D].             */
/* ------------------------------------------------------------------ */
void bzo_batch_prefill_ragged(const void* q, const void* k, const void* v, int dtype,
                              const int32_t* indptr, int B, int Hq, int Hkv, int D,
                              int causal, int rope, float rope_theta, float sm_scale,
                              const int32_t* rows, int n_rows, float* out) {
    const int G = Hq / Hkv;
    int N = indptr[B];
    int total = rows ? n_rows : N;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4)
#endif
    for (int ri = 0; ri < total; ++ri) {
        int i = rows ? rows[ri] : ri;
        float* qv = (float*)malloc(sizeof(float) * D);
        float* kr = (float*)malloc(sizeof(float) * D);
        int r = 0;
        while (r < B && !(i >= indptr[r] && i < indptr[r + 1])) ++r;
        float* obase = out + (size_t)ri * Hq * D;
        if (r == B) { memset(obase, 0, sizeof(float) * (size_t)Hq * D); free(qv); free(kr); continue; }
        int beg = indptr[r], end = causal ? i + 1 : indptr[r + 1];
        int L = end - beg;
        float* s = (float*)malloc(sizeof(float) * (size_t)L);
        for (int h = 0; h < Hq; ++h) {
            int kvh = h / G;
            float* o = obase + (size_t)h * D;
            for (int d = 0; d < D; ++d) { o[d] = 0.0f; qv[d] = load_as_f32(q, dtype, ((size_t)i * Hq + h) * D + d); }
            if (rope) bzo_rope_llama(qv, D, i - beg, rope_theta);
            float m = -INFINITY;
            for (int j = beg; j < end; ++j) {
                for (int d = 0; d < D; ++d) kr[d] = load_as_f32(k, dtype, ((size_t)j * Hkv + kvh) * D + d);
                if (rope == 1) bzo_rope_llama(kr, D, j - beg, rope_theta); /* rope == 2: k rows are rotated already */
                float acc = 0.0f;
                for (int d = 0; d < D; ++d) acc += qv[d] * kr[d];
                s[j - beg] = acc * sm_scale;
                if (s[j - beg] > m) m = s[j - beg];
            }
            float l = 0.0f;
            for (int j = beg; j < end; ++j) {
                float p = expf(s[j - beg] - m);
                l += p;
                for (int d = 0; d < D; ++d) o[d] += p * load_as_f32(v, dtype, ((size_t)j * Hkv + kvh) * D + d);
            }
            float inv = 1.0f / l;
            for (int d = 0; d < D; ++d) o[d] *= inv;
        }
        free(s); free(qv); free(kr);
    }
}

/* ------------------------------------------------------------------ */
/* KV page writes.  Pool is written in place through non-const aliases. */
/* src_dtype: dtype of the incoming k/v rows; the pool is kv->kv_dtype. */
/* When they differ (e4m3 pool) the value stored is                     */
/*   quant(x / scale[head]), scale NULL = 1.                            */
/* rope != 0: K rows are rotated (fp32) at their sequence position      */
/* before rounding to the pool dtype; V is never rotated.               */
/* ------------------------------------------------------------------ */
static void write_row(void* pool, int pool_dtype, int64_t off, const void* src, int src_dtype,
                      size_t soff, int D, int rope, int pos, float theta, float inv_scale_div,
                      int has_scale, float* tmp) {
    if (!rope && pool_dtype == src_dtype) { /* pure copy: bit exact */
        size_t es = dtype_size(pool_dtype);
        memcpy((char*)pool + (size_t)off * es, (const char*)src + soff * es, es * (size_t)D);
        return;
    }
    for (int d = 0; d < D; ++d) tmp[d] = load_as_f32(src, src_dtype, soff + d);
    if (rope) bzo_rope_llama(tmp, D, pos, theta);
    for (int d = 0; d < D; ++d) {
        float x = has_scale ? tmp[d] / inv_scale_div : tmp[d];
        store_from_f32(pool, pool_dtype, (size_t)(off + d), x);
    }
}

/* store_prefill_kv_cache (page.cu:21-94): token t < len_b of request b goes to page
 * indices[indptr[b] + t/P], slot t%P, all heads; sequence position starts at 0. */
void bzo_store_prefill_kv(const bzo_paged_kv* kv, const void* k, const void* v, int src_dtype,
                          const int32_t* ragged_indptr, int rope, float rope_theta,
                          const float* k_scale, const float* v_scale) {
    const int D = kv->head_dim, H = kv->num_kv_heads;
    float* tmp = (float*)malloc(sizeof(float) * D);
    for (int b = 0; b < kv->batch_size; ++b) {
        int len = ragged_indptr[b + 1] - ragged_indptr[b];
        for (int t = 0; t < len; ++t)
            for (int h = 0; h < H; ++h) {
                int64_t off = kv_elem_off(kv, b, t, h);
                size_t soff = ((size_t)(ragged_indptr[b] + t) * H + h) * D;
                write_row((void*)kv->k_base, kv->kv_dtype, off, k, src_dtype, soff, D, rope, t, rope_theta,
                          k_scale ? k_scale[h] : 1.0f, k_scale != NULL, tmp);
                write_row((void*)kv->v_base, kv->kv_dtype, off, v, src_dtype, soff, D, 0, 0, 0.0f,
                          v_scale ? v_scale[h] : 1.0f, v_scale != NULL, tmp);
            }
    }
    free(tmp);
}

/* append_decode_kv_cache (page.cu:96-115): one new row per sequence at position
 * seq_len-1, i.e. page indices[indptr[b+1]-1], slot last_page_len[b]-1. */
void bzo_append_decode_kv(const bzo_paged_kv* kv, const void* k, const void* v, int src_dtype,
                          int rope, float rope_theta, const float* k_scale, const float* v_scale) {
    const int D = kv->head_dim, H = kv->num_kv_heads;
    float* tmp = (float*)malloc(sizeof(float) * D);
    for (int b = 0; b < kv->batch_size; ++b) {
        int64_t L = seq_len_of(kv, b);
        if (L == 0) continue;
        for (int h = 0; h < H; ++h) {
            int64_t off = kv_elem_off(kv, b, L - 1, h);
            size_t soff = ((size_t)b * H + h) * D;
            write_row((void*)kv->k_base, kv->kv_dtype, off, k, src_dtype, soff, D, rope, (int)(L - 1), rope_theta,
                      k_scale ? k_scale[h] : 1.0f, k_scale != NULL, tmp);
            write_row((void*)kv->v_base, kv->kv_dtype, off, v, src_dtype, soff, D, 0, 0, 0.0f,
                      v_scale ? v_scale[h] : 1.0f, v_scale != NULL, tmp);
        }
    }
    free(tmp);
}

/* rotate decode q [B,Hq,D] in place at position seq_len_b-1, rounding to q's dtype */
void bzo_rope_decode_q_inplace(void* q, int dtype, const bzo_paged_kv* kv, int Hq, float theta) {
    const int D = kv->head_dim;
    float* row = (float*)malloc(sizeof(float) * D);
    for (int b = 0; b < kv->batch_size; ++b) {
        int64_t L = seq_len_of(kv, b);
        if (L == 0) continue;
        for (int h = 0; h < Hq; ++h) {
            size_t off = ((size_t)b * Hq + h) * D;
            for (int d = 0; d < D; ++d) row[d] = load_as_f32(q, dtype, off + d);
            bzo_rope_llama(row, D, (int)(L - 1), theta);
            for (int d = 0; d < D; ++d) store_from_f32(q, dtype, off + d, row[d]);
        }
    }
    free(row);
}

/* ------------------------------------------------------------------ */
/* element-wise ops.  *_f32 outputs are the unrounded fp32 values the   */
/* GPU result is compared with; storage outputs are RNE-rounded.        */
/* ------------------------------------------------------------------ */

/* rms_norm (rms_norm.h:11-19): out = x * rsqrt(mean(x^2) + eps) * w */
void bzo_rms_norm(const void* x, const void* w, int dtype, int N, int h, float eps, float* out_f32) {
    for (int n = 0; n < N; ++n) {
        float ss = 0.0f;
        for (int i = 0; i < h; ++i) { float a = load_as_f32(x, dtype, (size_t)n * h + i); ss += a * a; }
        float r = 1.0f / sqrtf(ss / (float)h + eps);
        for (int i = 0; i < h; ++i)
            out_f32[(size_t)n * h + i] = load_as_f32(x, dtype, (size_t)n * h + i) * r * load_as_f32(w, dtype, i);
    }
}

/* add_rms_norm (rms_norm.h:26-34): residual += input (rounded to storage);
 * input = rms_norm(residual) * w computed from the ROUNDED residual. */
void bzo_add_rms_norm(const void* input, void* residual, const void* w, int dtype, int N, int h, float eps,
                      float* out_f32) {
    for (int n = 0; n < N; ++n) {
        float ss = 0.0f;
        for (int i = 0; i < h; ++i) {
            size_t o = (size_t)n * h + i;
            float a = load_as_f32(input, dtype, o) + load_as_f32(residual, dtype, o);
            store_from_f32(residual, dtype, o, a);
            a = load_as_f32(residual, dtype, o);
            ss += a * a;
        }
        float r = 1.0f / sqrtf(ss / (float)h + eps);
        for (int i = 0; i < h; ++i) {
            size_t o = (size_t)n * h + i;
            out_f32[o] = load_as_f32(residual, dtype, o) * r * load_as_f32(w, dtype, i);
        }
    }
}

/* silu_and_mul (activation.h:7-16): out[n,i] = silu(in[n,i]) * in[n,I+i], gate first */
void bzo_silu_and_mul(const void* in, int dtype, int N, int I, float* out_f32) {
    for (int n = 0; n < N; ++n)
        for (int i = 0; i < I; ++i) {
            float g = load_as_f32(in, dtype, (size_t)n * 2 * I + i);
            float u = load_as_f32(in, dtype, (size_t)n * 2 * I + I + i);
            out_f32[(size_t)n * I + i] = g / (1.0f + expf(-g)) * u;
        }
}

/* exact sum of two storage values rounded ONCE to the storage type (ties to even): the fp32 sum of
 * two f16 values can itself be inexact, so the candidate from the float path is corrected against
 * its neighbours in double, where the sum is exact. */
static double bits16_to_f64(uint16_t b, int dtype) {
    return (double)(dtype == BZO_F16 ? bzo_f16_to_f32(b) : bzo_bf16_to_f32(b));
}
static uint16_t round_f64_to_16(double x, int dtype) {
    uint16_t c = (dtype == BZO_F16) ? bzo_f32_to_f16((float)x) : bzo_f32_to_bf16((float)x);
    if (x != x) return c;
    uint16_t best = c;
    double bd = fabs(bits16_to_f64(c, dtype) - x);
    for (int delta = -1; delta <= 1; delta += 2) {
        uint16_t mag = c & 0x7fffu;
        if (delta < 0 && mag == 0) continue;
        uint16_t n = (uint16_t)((c & 0x8000u) | (uint16_t)(mag + delta));
        double v = bits16_to_f64(n, dtype);
        if (isinf(v) || v != v) continue;
        double d = fabs(v - x);
        if (d < bd || (d == bd && !(n & 1u) && (best & 1u))) { best = n; bd = d; }
    }
    return best;
}

/* add_residual (add.h:8-14, add.cu:29-32): residual += input with ONE rounding to the
 * storage type per element (the half2 add rounds the exact sum once). */
void bzo_add_residual(const void* input, void* residual, int dtype, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        double s = (double)load_as_f32(input, dtype, i) + (double)load_as_f32(residual, dtype, i);
        ((uint16_t*)residual)[i] = round_f64_to_16(s, dtype);
    }
}

/* embedding (embedding.cu:7-47): out row (out_loc ? out_loc[t] : t) <- weight row token_ids[t] */
void bzo_embedding(uint16_t* out, const uint32_t* token_ids, const int32_t* out_loc, const uint16_t* weight,
                   size_t num_tokens, size_t hidden) {
    for (size_t t = 0; t < num_tokens; ++t) {
        const size_t d = out_loc ? (size_t)out_loc[t] : t;
        for (size_t i = 0; i < hidden; ++i) out[d * hidden + i] = weight[(size_t)token_ids[t] * hidden + i];
    }
}

/* gather_last_token (sampler.h:8-16): out row b <- tokens row ragged_indptr[b+1]-1, the whole row
 * (what the header documents; the reference's kernel drops the lane offset on the destination,
 * sampler.cu:21-24).  A request without tokens yields a zero row. */
void bzo_gather_last_token(uint16_t* out, const uint16_t* tokens, const int32_t* ragged_indptr, size_t batch,
                           size_t hidden) {
    for (size_t b = 0; b < batch; ++b)
        for (size_t i = 0; i < hidden; ++i)
            out[b * hidden + i] =
                ragged_indptr[b + 1] > ragged_indptr[b] ? tokens[(size_t)(ragged_indptr[b + 1] - 1) * hidden + i] : 0;
}

/* batch_find_max (sampler.h:18-26): argmax of each row: the smallest index of the largest non-NaN
 * value, 0 if the row has none (sampler.cu:87-108 leaves ties to a race and starts from -65400). */
void bzo_batch_find_max(uint32_t* out, const void* input, int dtype, size_t batch, size_t length) {
    for (size_t b = 0; b < batch; ++b) {
        float best = 0.f;
        int have = 0;
        uint32_t bi = 0;
        for (size_t i = 0; i < length; ++i) {
            const float v = load_as_f32(input, dtype, b * length + i);
            if (v != v) continue;
            if (!have || v > best) { best = v; bi = (uint32_t)i; have = 1; }
        }
        out[b] = bi;
    }
}

/* ------------------------------------------------------------------ */
/* host page table logic                                                */
/* ------------------------------------------------------------------ */

/* prefill reservation (batch.h:236-257): a request of len tokens reserves len+1 slots */
void bzo_prefill_reservation(const int32_t* lens, int B, int P, int32_t* indptr /*[B+1]*/,
                             int32_t* last_page_len /*[B]*/) {
    int32_t acc = 0;
    for (int b = 0; b < B; ++b) {
        int32_t need_slots = lens[b] + 1;
        int32_t need_blocks = (need_slots + P - 1) / P;
        indptr[b] = acc;
        acc += need_blocks;
        last_page_len[b] = need_slots - (need_blocks - 1) * P;
    }
    indptr[B] = acc;
}

/* first-fit lowest free ids (cache_manager.h:161-184); returns count found */
int bzo_first_fit(uint8_t* free_mask, int max_pages, int n, int32_t* out) {
    int cnt = 0;
    for (int i = 0; i < max_pages && cnt < n; ++i)
        if (free_mask[i]) out[cnt++] = i;
    if (cnt < n) return cnt; /* caller treats as allocation failure; mask untouched */
    for (int i = 0; i < n; ++i) free_mask[out[i]] = 0;
    return cnt;
}

/* ------------------------------------------------------------------ */
/* Row-major strided-batched GEMM with the argument meaning of          */
/* util::CublasWrapper::gemmStridedBatched (src/util/cublas_wrapper.h:  */
/* 33-88; operand swap for the column-major library at :183-207):       */
/*   C[b] (m x n, ld n) = alpha * op(A[b]) * op(B[b]) + beta * C[b]     */
/*   A[b] stored m x k (ld k) if !transa else k x m (ld m)              */
/*   B[b] stored k x n (ld n) if !transb else n x k (ld k)              */
/* fp32 accumulation in index order, alpha and beta applied in fp32,    */
/* one rounding to the storage type.  (The reference asks cuBLAS for    */
/* fp16 accumulation on half, :144-146; fp32 is the stricter checker.)  */
/* ------------------------------------------------------------------ */
void bzo_gemm_strided_batched(int transa, int transb, int m, int n, int k, float alpha, const void* A,
                              int64_t stride_a, const void* B, int64_t stride_b, float beta, void* C,
                              int64_t stride_c, int batch, int dtype) {
    const size_t es = dtype_size(dtype);
    for (int b = 0; b < batch; ++b) {
        const char* Ab = (const char*)A + (size_t)b * (size_t)stride_a * es;
        const char* Bb = (const char*)B + (size_t)b * (size_t)stride_b * es;
        char* Cb = (char*)C + (size_t)b * (size_t)stride_c * es;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
        for (int r = 0; r < m; ++r)
            for (int c = 0; c < n; ++c) {
                float acc = 0.0f;
                for (int i = 0; i < k; ++i) {
                    const float a = load_as_f32(Ab, dtype, transa ? (size_t)i * m + r : (size_t)r * k + i);
                    const float bb = load_as_f32(Bb, dtype, transb ? (size_t)c * k + i : (size_t)i * n + c);
                    acc += a * bb;
                }
                float v = alpha * acc;
                if (beta != 0.0f) v += beta * load_as_f32(Cb, dtype, (size_t)r * n + c);
                store_from_f32(Cb, dtype, (size_t)r * n + c, v);
            }
    }
}

/* number of threads the parallel build uses (1 for the scalar build) */
#ifdef _OPENMP
#include <omp.h>
int bzo_num_threads(void) { return omp_get_max_threads(); }
#else
int bzo_num_threads(void) { return 1; }
#endif

/* one decode step of page-table growth (cache_manager.h:255-324): a sequence whose last page is full
 * gets the next lowest free page and restarts at slot 1, every other sequence gains one slot.
 * indices must have room for B more entries.  Returns the new number of pages, or -1 (nothing
 * changed) when the pool cannot supply the pages -- the reference throws at that point with the
 * slot counts already bumped (cache_manager.h:264-281); all-or-nothing is the contract checked here. */
int bzo_table_grow(int32_t* indices, int32_t* indptr, int32_t* last_page_len, int B, int P, uint8_t* free_mask,
                   int max_pages) {
    int nfull = 0;
    for (int i = 0; i < B; ++i) nfull += (last_page_len[i] == P);
    int32_t* fresh = (int32_t*)malloc(sizeof(int32_t) * (size_t)(nfull > 0 ? nfull : 1));
    if (bzo_first_fit(free_mask, max_pages, nfull, fresh) < nfull) { free(fresh); return -1; }
    int nnz = indptr[B];
    int32_t* out = (int32_t*)malloc(sizeof(int32_t) * (size_t)(nnz + nfull + 1));
    int w = 0, f = 0, start = 0;
    for (int i = 0; i < B; ++i) {
        int end = indptr[i + 1];
        for (int j = start; j < end; ++j) out[w++] = indices[j];
        start = end;
        if (last_page_len[i] == P) { out[w++] = fresh[f++]; last_page_len[i] = 1; }
        else last_page_len[i] += 1;
        indptr[i + 1] = w;
    }
    memcpy(indices, out, sizeof(int32_t) * (size_t)w);
    free(out); free(fresh);
    return w;
}
