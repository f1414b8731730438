// What the matrix pipes of this GPU sustain: v_mfma_f32_32x32x16_f16 at full rate, two waves per SIMD, 256
// workgroups of 512 threads, no memory traffic at all -- on operands of constant bits, on random operands, and
// with what an attention kernel must do beside every matrix instruction (a 1 KiB operand read from LDS, an
// exponential, half a pack and half a row-sum instruction), each perfectly overlapped.  The clock is read on
// the device (shader cycles over wall time), because the chip lowers it under this load: the figures are what
// the power limit leaves of the 2.5 PFLOP/s that the data sheet quotes at 2.4 GHz.  Prints one line per variant;
// bench.py --workload MFMA_CEILING runs this program and reports the lines.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef uint32_t __attribute__((ext_vector_type(4))) u32x4;
typedef __attribute__((ext_vector_type(2))) _Float16 h2;
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("hip error %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
// MODE bit 0: A operand of every MFMA read from LDS (ds_read_b128, conflict free); bit 1: 1 exp + 0.5 pack + 0.5 dot2 per MFMA;
// bit 2: A operands of every second MFMA only (reuse); bit 3: operands of constant bits instead of random ones
template <int MODE>
__global__ __launch_bounds__(512) void k(int iters, float* out, const unsigned* rnd) {
    extern __shared__ unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) ((unsigned*)smem)[i] = rnd[i & 32767] & 0x3fff3fffu; // small halves
    __syncthreads();
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
    f32x16 acc[4];
    for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    f16x8 a[8], b[8];
    for (int i = 0; i < 8; ++i)
        for (int e = 0; e < 8; ++e) {
            unsigned r = rnd[(threadIdx.x * 8 + i) * 8 + e];
            a[i][e] = (MODE & 8) ? (_Float16)1.0f : (_Float16)(((int)(r & 0xffff) - 32768) * (1.0f / 16384.f));
            b[i][e] = (MODE & 8) ? (_Float16)1.0f : (_Float16)(((int)(r >> 16) - 32768) * (1.0f / 16384.f));
        }
    float y[16]; for (int e = 0; e < 16; ++e) y[e] = -0.01f * (lane + e);
    float psum = 0.f; unsigned pk[8] = {0};
    const uint32_t addr = lds0 + (wave & 7) * 8192 + lane * 16;
    u32x4 ring[4];
    for (int i = 0; i < 4; ++i) ring[i] = *reinterpret_cast<const u32x4 __attribute__((address_space(3)))*>((const unsigned char __attribute__((address_space(3)))*)(uintptr_t)(addr) + i * 1024);
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (MODE & 1) {
                f16x8 av = __builtin_bit_cast(f16x8, ring[u & 3]);
                acc[u & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, b[(u * 3) & 7], acc[u & 3], 0, 0, 0);
                if (!(MODE & 4) || (u & 1))
                    ring[u & 3] = *reinterpret_cast<const u32x4 __attribute__((address_space(3)))*>((const unsigned char __attribute__((address_space(3)))*)(uintptr_t)(addr) + ((u + it) & 7) * 1024);
            } else {
                acc[u & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[u & 7], b[(u * 3) & 7], acc[u & 3], 0, 0, 0);
            }
            if (MODE & 2) {
                y[u] = __builtin_amdgcn_exp2f(y[u] * 0.999f);
                if (u & 1) {
                    h2 hw = __builtin_convertvector((__attribute__((ext_vector_type(2))) float){y[u - 1], y[u]}, h2);
                    pk[u >> 1] = __builtin_bit_cast(unsigned, hw);
                    psum = __builtin_amdgcn_fdot2(hw, h2{(_Float16)1.0f, (_Float16)1.0f}, psum, false);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float r = psum;
    for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) r += acc[j][e];
    for (int e = 0; e < 16; ++e) r += y[e];
    for (int e = 0; e < 8; ++e) r += pk[e];
    if (r == 123.456f) out[lane] = r;
    if (threadIdx.x == 0 && blockIdx.x == 0) { ((long long*)out)[64] = c1 - c0; ((long long*)out)[65] = w1 - w0; }
}
template <int MODE>
void run(const char* name, float* out, const unsigned* rnd) {
    const int iters = 40000;
    hipEvent_t e0, e1; CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    CHECK(hipFuncSetAttribute((const void*)k<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    k<MODE><<<256, 512, 65536>>>(1000, out, rnd);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0));
    k<MODE><<<256, 512, 65536>>>(iters, out, rnd);
    CHECK(hipEventRecord(e1));
    CHECK(hipDeviceSynchronize());
    float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
    long long h[2]; CHECK(hipMemcpy(h, (char*)out + 512, 16, hipMemcpyDeviceToHost));
    const double flops = 256.0 * 8 * iters * 16 * 32768.0;
    const double clk = (double)h[0] / ((double)h[1] / 100.0);
    printf("%-52s %8.2f ms  %7.1f TFLOP/s  clock %.0f MHz  pipe use %.0f %%\n", name, ms, flops / ms / 1e9, clk,
           100.0 * (flops / ms / 1e9) / (2500.0 * clk / 2400.0));
    fflush(stdout);
}
int main() {
    float* out; CHECK(hipMalloc(&out, 4096));
    unsigned* rnd; CHECK(hipMalloc(&rnd, 32768 * 4));
    unsigned* hr = (unsigned*)malloc(32768 * 4);
    srand(1); for (int i = 0; i < 32768; ++i) hr[i] = ((unsigned)rand() << 16) ^ (unsigned)rand();
    CHECK(hipMemcpy(rnd, hr, 32768 * 4, hipMemcpyHostToDevice));
    for (int rep = 0; rep < 2; ++rep) {
        run<8>("matrix only, operands of constant bits", out, rnd);
        run<0>("matrix only, random operands (registers)", out, rnd);
        run<1>("+ A operand from LDS, every instruction", out, rnd);
        run<5>("+ A operand from LDS, every second instruction", out, rnd);
        run<2>("+ exp, pack, dot2 (registers)", out, rnd);
        run<3>("+ LDS every instruction + exp, pack, dot2", out, rnd);
        run<7>("+ LDS every second + exp, pack, dot2", out, rnd);
    }
    return 0;
}
