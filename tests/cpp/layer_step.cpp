// One Llama-2-7B-shaped decoder layer (hidden 4096, 32 heads, intermediate 11008) stepping a decode
// batch of 64 sequences through the C++ drop-in headers with every GEMM on hipBLASLt: the "single-layer decode step" of
// a Llama-2-7B decode benchmark with the four GEMMs in.  Checks
//   1. blitz::util::HipblasLtGemm, in every call form of the reference's GEMM wrapper, against the CPU checker's GEMM,
//   2. the layer's residual stream against the same layer run with a naive one-thread-per-element GEMM,
// and prints the time of a layer step.  Runs on the GPU box; built without a GPU.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include <hip/hip_runtime.h>

#include "blitz/cache_manager.h"
#include "kernel/attention.h"
#include "layer/attn.h"
#include "layer/glu.h"
#include "util/hipblaslt_gemm.h"

#define HIP_OK(x)                                                                         \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            exit(2);                                                                      \
        }                                                                                 \
    } while (0)

using half_t = __half;

// naive row-major GEMM, fp32 accumulate in index order, one rounding to f16: test infrastructure only
__global__ void naive_gemm(int m, int n, int k, const __half* A, const __half* B, __half* C) {
    const int col = blockIdx.x * blockDim.x + threadIdx.x, row = blockIdx.y;
    if (col >= n) return;
    float acc = 0.f;
    for (int i = 0; i < k; ++i) acc += __half2float(A[(size_t)row * k + i]) * __half2float(B[(size_t)i * n + col]);
    C[(size_t)row * n + col] = __float2half_rn(acc);
}
struct NaiveGemm : blitz::util::GemmWrapper {
    using GemmWrapper::gemmStridedBatched;
    void gemmStridedBatched(blitz::util::GemmOp ta, blitz::util::GemmOp tb, int m, int n, int k, float alpha, const void* A,
                            long long int, const void* B, long long int, float beta, void* C, long long int,
                            int batch) override {
        if (ta != blitz::util::GemmOp::N || tb != blitz::util::GemmOp::N || alpha != 1.f || beta != 0.f || batch != 1) {
            printf("NaiveGemm: only the plain product the layers call\n");
            exit(5);
        }
        hipLaunchKernelGGL(naive_gemm, dim3((n + 127) / 128, m), dim3(128), 0, 0, m, n, k, (const __half*)A,
                           (const __half*)B, (__half*)C);
    }
};
// the CPU checker's GEMM (oracle/bz_oracle.c): fp32 accumulation in index order, one rounding
extern "C" void bzo_gemm_strided_batched(int transa, int transb, int m, int n, int k, float alpha, const void* A,
                                         int64_t stride_a, const void* B, int64_t stride_b, float beta, void* C,
                                         int64_t stride_c, int batch, int dtype);
// device fill: uniform(-scale, scale) + mean from a counter hash (no host buffers of gigabytes)
__global__ void fill_uniform(__half* p, size_t n, float scale, float mean, uint64_t seed) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        p[i] = __float2half_rn(mean + scale * (float)((double)(z >> 11) / 9007199254740992.0 * 2.0 - 1.0));
    }
}
static void fill(__half* p, size_t n, float scale, float mean, uint64_t seed) {
    hipLaunchKernelGGL(fill_uniform, dim3(2048), dim3(256), 0, 0, p, n, scale, mean, seed);
}
static double max_abs_diff_dev(const __half* a, const __half* b, size_t n, double* max_ref) {
    std::vector<__half> ha(n), hb(n);
    HIP_OK(hipMemcpy(ha.data(), a, n * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(hb.data(), b, n * 2, hipMemcpyDeviceToHost));
    double m = 0, r = 0;
    for (size_t i = 0; i < n; ++i) {
        const double x = __half2float(ha[i]), y = __half2float(hb[i]);
        if (!(x == x) || !(y == y)) return INFINITY;
        m = fmax(m, fabs(x - y));
        r = fmax(r, fabs(y));
    }
    if (max_ref) *max_ref = r;
    return m;
}

int main() {
    bool ok = true;
    blitz::util::HipblasLtGemm lt(HIP_R_16F);
    NaiveGemm naive;

    // ---- 1. the GEMM wrapper against the CPU checker's GEMM: every call form of the reference's wrapper
    // (src/util/cublas_wrapper.h:71-131) -- transposes, alpha/beta, strided batches -- on shapes the layers use
    // (inputs O(1)/sqrt(k): results O(1))
    using blitz::util::GemmOp;
    struct Case { int m, n, k, ta, tb, batch; float alpha, beta; int pad; };
    const Case cases[] = {
        {64, 512, 256, 0, 0, 1, 1.f, 0.f, 0},    {7, 1024, 384, 0, 0, 1, 1.f, 0.f, 0},
        {1, 4096, 4096, 0, 0, 1, 1.f, 0.f, 0},   {64, 4096, 4096, 0, 0, 1, 1.f, 0.f, 0},   // a 7B projection at batch 64
        {57, 264, 128, 0, 0, 1, 1.f, 0.f, 0},    {33, 136, 72, 1, 0, 1, 1.f, 0.f, 0},
        {33, 136, 72, 0, 1, 1, 1.f, 0.f, 0},     {33, 136, 72, 1, 1, 1, 0.5f, 0.f, 0},
        {16, 128, 64, 0, 0, 5, 1.f, 0.f, 0},     {16, 128, 64, 0, 1, 3, 2.f, -1.f, 24},    // batched, strides padded by 24 elements
        {40, 96, 200, 1, 0, 4, 1.f, 0.25f, 8},
    };
    for (const Case& c : cases) {
        const int m = c.m, n = c.n, k = c.k;
        const long long sa = (long long)m * k + c.pad, sb = (long long)k * n + c.pad, sc = (long long)m * n + c.pad;
        const size_t na = (size_t)sa * c.batch, nb = (size_t)sb * c.batch, nc = (size_t)sc * c.batch;
        __half *A, *B, *C1;
        HIP_OK(hipMalloc(&A, na * 2));
        HIP_OK(hipMalloc(&B, nb * 2));
        HIP_OK(hipMalloc(&C1, nc * 2));
        fill(A, na, 1.0f, 0.f, 11);
        fill(B, nb, 1.7f / sqrtf((float)k), 0.f, 12);
        fill(C1, nc, 1.0f, 0.f, 13); // previous contents of C: read when beta != 0, and the padding must survive
        std::vector<__half> hA(na), hB(nb), hC(nc), got(nc);
        HIP_OK(hipMemcpy(hA.data(), A, na * 2, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(hB.data(), B, nb * 2, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(hC.data(), C1, nc * 2, hipMemcpyDeviceToHost));
        const GemmOp ta = c.ta ? GemmOp::T : GemmOp::N, tb = c.tb ? GemmOp::T : GemmOp::N;
        if (c.batch == 1 && c.alpha == 1.f && c.beta == 0.f) lt.gemm(ta, tb, m, n, k, A, B, C1);
        else if (c.pad == 0 && c.alpha == 1.f && c.beta == 0.f) lt.gemmBatched(ta, tb, m, n, k, A, B, C1, c.batch);
        else lt.gemmStridedBatched(ta, tb, m, n, k, c.alpha, A, sa, B, sb, c.beta, C1, sc, c.batch);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(got.data(), C1, nc * 2, hipMemcpyDeviceToHost));
        bzo_gemm_strided_batched(c.ta, c.tb, m, n, k, c.alpha, hA.data(), sa, hB.data(), sb, c.beta, hC.data(), sc, c.batch, 0);
        double e = 0, ref = 0;
        bool pad_ok = true;
        for (size_t i = 0; i < nc; ++i) {
            const double x = __half2float(got[i]), y = __half2float(hC[i]);
            if ((long long)(i % (size_t)sc) >= (long long)m * n) { pad_ok = pad_ok && x == y; continue; }
            e = fmax(e, fabs(x - y));
            ref = fmax(ref, fabs(y));
            if (!(x == x)) e = INFINITY;
        }
        // both accumulate in fp32 and round once; the summation order differs: a few f16 steps at |c| ~ 2
        const bool good = e <= 4e-3 * fmax(1.0, ref) && pad_ok;
        printf("gemm %c%c %5d x %5d x %5d, batch %d, alpha %.2f beta %.2f: max |hipblaslt - cpu checker| = %.3e (max |c| %.2f) %s\n",
               c.ta ? 'T' : 'N', c.tb ? 'T' : 'N', m, n, k, c.batch, c.alpha, c.beta, e, ref, good ? "ok" : "BAD");
        ok = ok && good;
        (void)hipFree(A); (void)hipFree(B); (void)hipFree(C1);
    }

    // ---- 2. a Llama-2-7B-shaped layer, decode batch of 64, contexts U[512, 2048]
    const uint32_t hidden = 4096, Hq = 32, Hkv = 32, D = 128, inter = 11008, P = 16, B = 64;
    blitz::kernel::attention_options().rope_theta = 1e4f;
    std::vector<int32_t> lens(B);
    uint64_t st = 0x5EED;
    uint32_t need = 0;
    for (auto& l : lens) {
        st = st * 6364136223846793005ull + 1442695040888963407ull;
        l = 512 + (int32_t)((st >> 33) % 1537);
        need += (l + 2 + P - 1) / P;
    }
    const uint32_t max_pages = need + 16;
    blitz::CacheManager<half_t, int32_t> cm(Hkv, 1, D, P, max_pages, BZ_LAYOUT_HND, true, 1 << 20);
    fill((half_t*)cm.get_base_ptr(), (size_t)max_pages * 2 * Hkv * P * D, 1.0f, 0.f, 21); // a context of N(0,~0.58) keys/values
    blitz::HostBatch<half_t, int32_t> batch(&cm, lens); // reserves len+1 slots: a batch right after its prefill
    auto& pt = batch.page_table;
    cm.set_layer(pt, 0);
    int32_t* table_d;
    HIP_OK(hipMalloc(&table_d, 4 << 20));
    const size_t tn = pt.indices.size() + pt.indptr.size() + pt.last_page_len.size();
    HIP_OK(hipMemcpy(table_d, pt.indices_h, tn * 4, hipMemcpyHostToDevice));
    pt.indices_d = table_d;
    pt.indptr_d = table_d + pt.indices.size();
    pt.last_page_len_d = pt.indptr_d + pt.indptr.size();

    const size_t attn_w = hidden + 2 * (size_t)Hq * D * hidden + 2 * (size_t)Hkv * D * hidden;
    const size_t glu_w = hidden + 3 * (size_t)hidden * inter;
    half_t* w_d;
    HIP_OK(hipMalloc(&w_d, (attn_w + glu_w) * 2));
    fill(w_d, attn_w + glu_w, 1.7f / sqrtf((float)hidden), 0.f, 31);
    fill(w_d, hidden, 0.02f, 1.0f, 32);          // input norm
    fill(w_d + attn_w, hidden, 0.02f, 1.0f, 33); // post-attention norm
    void *float_ws, *int_ws;
    HIP_OK(hipMalloc(&float_ws, 128 << 20));
    HIP_OK(hipMalloc(&int_ws, 8 << 20));
    blitz::kernel::BatchPrefillRaggedHandler<half_t, int32_t> prefill_h(blitz::kernel::create_flashinfer_prefill_handler());
    blitz::kernel::BlitzBatchDecodeHandler<half_t, int32_t> decode_h(blitz::kernel::create_flashinfer_decode_handler());
    const size_t ws_elems = (size_t)B * (hidden + 3 * (size_t)std::max<uint32_t>(hidden, inter) + (size_t)(2 * Hq + 2 * Hkv) * D);
    half_t *ws_lt, *ws_nv, *x_d;
    HIP_OK(hipMalloc(&ws_lt, ws_elems * 2));
    HIP_OK(hipMalloc(&ws_nv, ws_elems * 2));
    HIP_OK(hipMalloc(&x_d, (size_t)B * hidden * 2));
    fill(x_d, (size_t)B * hidden, 1.7f, 0.f, 41);
    decode_h.plan(float_ws, 128 << 20, int_ws, 8 << 20, pt.indptr_h, pt.last_page_len_h, B, Hq, Hkv, D, P);

    auto run_layer = [&](blitz::util::GemmWrapper* g, half_t* ws) {
        half_t* seg = w_d;
        blitz::layer::Attention<half_t, int32_t> attn(g, &prefill_h, &decode_h, D, hidden, Hq, Hkv, ws, &seg);
        blitz::layer::GatedLinearUnit<half_t> glu(g, hidden, inter, ws, &seg);
        HIP_OK(hipMemcpy(ws, x_d, (size_t)B * hidden * 2, hipMemcpyDeviceToDevice));
        attn.forward(B, nullptr, pt);
        glu.forward(B);
        HIP_OK(hipDeviceSynchronize());
    };
    // both runs append the same new K/V at the same slot, so the second one sees the pool the first one left
    run_layer(&naive, ws_nv);
    run_layer(&lt, ws_lt);
    double ref = 0;
    const double e = max_abs_diff_dev(ws_lt, ws_nv, (size_t)B * hidden, &ref);
    const bool good = e <= 2e-2 * fmax(1.0, ref);
    printf("layer decode step, residual stream: max |hipblaslt - naive gemm| = %.3e (max |x| %.2f) %s\n", e, ref, good ? "ok" : "BAD");
    ok = ok && good;

    // ---- time of a layer step (events on the null stream, which everything here uses)
    {
        half_t* seg = w_d;
        blitz::layer::Attention<half_t, int32_t> attn(&lt, &prefill_h, &decode_h, D, hidden, Hq, Hkv, ws_lt, &seg);
        blitz::layer::GatedLinearUnit<half_t> glu(&lt, hidden, inter, ws_lt, &seg);
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        const int warm = 10, steps = 100;
        for (int i = 0; i < warm + steps; ++i) {
            if (i == warm) HIP_OK(hipEventRecord(e0, 0));
            attn.forward(B, nullptr, pt);
            glu.forward(B);
        }
        HIP_OK(hipEventRecord(e1, 0));
        HIP_OK(hipEventSynchronize(e1));
        float ms = 0;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        const double weights = (double)(attn_w + glu_w) * 2;
        printf("layer decode step (B 64, ctx U[512,2048], 7B shapes, all GEMMs on hipBLASLt): %.1f us; weights %.1f MB -> %.0f GB/s "
               "if the step were only the weight stream\n", ms * 1e3 / steps, weights / 1e6, weights / (ms * 1e-3 / steps) / 1e9);
    }
    printf(ok ? "PASS\n" : "FAIL\n");
    return ok ? 0 : 1;
}
