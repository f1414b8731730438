// Row-wise element-wise kernels for gfx950: RMSNorm, fused add+RMSNorm, SiLU-gate and residual
// add.  Replace src/kernel/norm.cu, activation.cu and add.cu of the BlitzScale worker.  All of
// them move 16 bytes per lane and reduce in fp32 with wave64 shuffles.
#include "bz_common.hpp"

namespace bz {

// sum over the workgroup; every lane gets the result
__device__ __forceinline__ float block_sum(float v, float* smem /* [16] */) {
    v = wave_sum(v);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, nw = (blockDim.x + 63) / 64;
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < nw; ++w) t += smem[w];
    __syncthreads();
    return t;
}

// out[n,:] = x[n,:] * rsqrt(mean(x^2)+eps) * w.  ADD: residual += input first (rounded to storage),
// x is the rounded residual and the result overwrites input.
template <typename T, bool ADD>
__global__ __launch_bounds__(1024) void rms_norm_kernel(T* input, T* residual, const T* weight, T* output,
                                                         uint32_t h, float eps) {
    __shared__ float smem[16];
    const size_t row = (size_t)blockIdx.x * h;
    const uint32_t nvec = h / 8;
    float ss = 0.f;
    for (uint32_t i = threadIdx.x; i < nvec; i += blockDim.x) {
        Vec8<T> v;
        float x[8];
        v.load(input + row + i * 8);
        v.to_float(x);
        if (ADD) {
            Vec8<T> r;
            float y[8];
            r.load(residual + row + i * 8);
            r.to_float(y);
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] += y[e];
            r.from_float(x);
            r.store(residual + row + i * 8);
            r.to_float(x); // the rounded residual is what gets normalised
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
    }
    ss = block_sum(ss, smem);
    const float rr = rsqrtf(ss / (float)h + eps);
    const T* src = ADD ? residual : input;
    for (uint32_t i = threadIdx.x; i < nvec; i += blockDim.x) {
        Vec8<T> v, w;
        float x[8], g[8];
        v.load(src + row + i * 8);
        w.load(weight + i * 8);
        v.to_float(x);
        w.to_float(g);
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = x[e] * rr * g[e];
        v.from_float(x);
        v.store(output + row + i * 8);
    }
}

// out[n,i] = silu(in[n,i]) * in[n,I+i]
template <typename T>
__global__ __launch_bounds__(256) void silu_and_mul_kernel(const T* in, T* out, uint32_t I) {
    const size_t n = blockIdx.y;
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= I) return;
    Vec8<T> g, u;
    float gf[8], uf[8];
    g.load(in + n * 2 * I + i);
    u.load(in + n * 2 * I + I + i);
    g.to_float(gf);
    u.to_float(uf);
#pragma unroll
    for (int e = 0; e < 8; ++e) gf[e] = gf[e] / (1.0f + __expf(-gf[e])) * uf[e];
    g.from_float(gf);
    g.store(out + n * I + i);
}

// residual += input, exactly one rounding per element
template <typename T> __device__ __forceinline__ void add8(Vec8<T>& r, const Vec8<T>& x);
template <> __device__ __forceinline__ void add8<f16_t>(Vec8<f16_t>& r, const Vec8<f16_t>& x) {
    // native packed f16 add rounds the exact sum once
    uint32_t a[4] = {r.raw.x, r.raw.y, r.raw.z, r.raw.w};
    const uint32_t b[4] = {x.raw.x, x.raw.y, x.raw.z, x.raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        __half2 ha = *reinterpret_cast<__half2*>(&a[i]);
        const __half2 hb = *reinterpret_cast<const __half2*>(&b[i]);
        ha = __hadd2(ha, hb);
        a[i] = *reinterpret_cast<uint32_t*>(&ha);
    }
    r.raw = make_uint4(a[0], a[1], a[2], a[3]);
}
template <> __device__ __forceinline__ void add8<bf16_t>(Vec8<bf16_t>& r, const Vec8<bf16_t>& x) {
    // the fp32 sum of two bf16 values is exact whenever it can matter for the bf16 rounding
    float a[8], b[8];
    r.to_float(a);
    x.to_float(b);
#pragma unroll
    for (int e = 0; e < 8; ++e) a[e] += b[e];
    r.from_float(a);
}

template <typename T>
__global__ __launch_bounds__(256) void add_residual_kernel(const T* input, T* residual, size_t nvec) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nvec) return;
    Vec8<T> r, x;
    r.load(residual + i * 8);
    x.load(input + i * 8);
    add8<T>(r, x);
    r.store(residual + i * 8);
}

static inline uint32_t norm_block(uint32_t h) {
    uint32_t t = (h / 8 + 63) / 64 * 64;
    if (t > 1024) t = 1024;
    if (t < 64) t = 64;
    return t;
}

} // namespace bz

using namespace bz;

extern "C" int bz_rms_norm(const void* input, const void* weight, void* output, int dtype, uint32_t num_tokens,
                           uint32_t hidden_size, float eps, void* stream) {
    if (!input || !weight || !output) return BZ_ERR_BAD_ARG;
    if (hidden_size % 8) return BZ_ERR_UNSUPPORTED;
    if (num_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(num_tokens), block(norm_block(hidden_size));
    if (dtype == BZ_F16)
        hipLaunchKernelGGL((rms_norm_kernel<f16_t, false>), grid, block, 0, s, (f16_t*)input, (f16_t*)nullptr,
                           (const f16_t*)weight, (f16_t*)output, hidden_size, eps);
    else if (dtype == BZ_BF16)
        hipLaunchKernelGGL((rms_norm_kernel<bf16_t, false>), grid, block, 0, s, (bf16_t*)input, (bf16_t*)nullptr,
                           (const bf16_t*)weight, (bf16_t*)output, hidden_size, eps);
    else return BZ_ERR_UNSUPPORTED;
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_add_rms_norm(void* input, void* residual, const void* weight, int dtype, uint32_t num_tokens,
                               uint32_t hidden_size, float eps, void* stream) {
    if (!input || !weight || !residual) return BZ_ERR_BAD_ARG;
    if (hidden_size % 8) return BZ_ERR_UNSUPPORTED;
    if (num_tokens == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(num_tokens), block(norm_block(hidden_size));
    if (dtype == BZ_F16)
        hipLaunchKernelGGL((rms_norm_kernel<f16_t, true>), grid, block, 0, s, (f16_t*)input, (f16_t*)residual,
                           (const f16_t*)weight, (f16_t*)input, hidden_size, eps);
    else if (dtype == BZ_BF16)
        hipLaunchKernelGGL((rms_norm_kernel<bf16_t, true>), grid, block, 0, s, (bf16_t*)input, (bf16_t*)residual,
                           (const bf16_t*)weight, (bf16_t*)input, hidden_size, eps);
    else return BZ_ERR_UNSUPPORTED;
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_silu_and_mul(const void* input, void* output, int dtype, uint32_t num_tokens, uint32_t inter_size,
                               void* stream) {
    if (!input || !output) return BZ_ERR_BAD_ARG;
    if (inter_size % 8) return BZ_ERR_UNSUPPORTED;
    if (num_tokens == 0 || inter_size == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 block(256), grid((inter_size / 8 + 255) / 256, num_tokens);
    if (dtype == BZ_F16)
        hipLaunchKernelGGL((silu_and_mul_kernel<f16_t>), grid, block, 0, s, (const f16_t*)input, (f16_t*)output, inter_size);
    else if (dtype == BZ_BF16)
        hipLaunchKernelGGL((silu_and_mul_kernel<bf16_t>), grid, block, 0, s, (const bf16_t*)input, (bf16_t*)output, inter_size);
    else return BZ_ERR_UNSUPPORTED;
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_add_residual(const void* input, void* residual, int dtype, uint32_t num_tokens, uint32_t dim,
                               void* stream) {
    if (!input || !residual) return BZ_ERR_BAD_ARG;
    const size_t n = (size_t)num_tokens * dim;
    if (n % 8) return BZ_ERR_UNSUPPORTED;
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t nvec = n / 8;
    const dim3 block(256), grid((unsigned)((nvec + 255) / 256));
    if (dtype == BZ_F16)
        hipLaunchKernelGGL((add_residual_kernel<f16_t>), grid, block, 0, s, (const f16_t*)input, (f16_t*)residual, nvec);
    else if (dtype == BZ_BF16)
        hipLaunchKernelGGL((add_residual_kernel<bf16_t>), grid, block, 0, s, (const bf16_t*)input, (bf16_t*)residual, nvec);
    else return BZ_ERR_UNSUPPORTED;
    BZ_LAUNCH_CHECK();
    return 0;
}
