// Row gathers and greedy sampling of the decode loop: replaces src/kernel/embedding.cu and
// src/kernel/sampler.cu of the BlitzScale worker.  All three are HBM-bound copies/reductions over
// rows of 16-bit elements; rows move 16 bytes per lane.
//
//   embedding ........... out[loc(t)] = weight[token_ids[t]]            (embedding.cu:7-47)
//   gather_last_token ... out[b] = tokens[ragged_indptr[b+1] - 1]       (sampler.cu:7-25)
//   batch_find_max ...... out[b] = argmax_i input[b][i]                 (sampler.cu:80-109)
//
// Two things the reference gets wrong are not reproduced: its gather copies every lane's 16 bytes to
// the start of the output row (sampler.cu:21-24 lacks the lane offset on the destination), and its
// argmax leaves the index undefined when no element exceeds -65400 and lets any lane holding the
// maximum write its index (ties resolved by a race, sampler.cu:87-108).  Here the whole row is copied
// and argmax is the smallest index of the largest non-NaN value (0 for a row without one).
#include <cmath>

#include "bz_common.hpp"

namespace bz {

// grid (rows), block 256: row r of dst <- row src_row(r) of src, hidden % 8 == 0 elements of 2 bytes
__global__ __launch_bounds__(256) void gather_rows_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                           const uint32_t* __restrict__ token_ids,
                                                           const int32_t* __restrict__ out_loc,
                                                           const int32_t* __restrict__ ragged_indptr,
                                                           uint32_t row_vecs) {
    const uint32_t r = blockIdx.x;
    int64_t s, d = r;
    if (ragged_indptr) { // last token of request r; a request without tokens yields a zero row
        s = (int64_t)ragged_indptr[r + 1] - 1;
        if (ragged_indptr[r + 1] <= ragged_indptr[r]) s = -1;
    } else {
        s = token_ids[r];
        if (out_loc) d = out_loc[r];
    }
    uint4* drow = dst + (size_t)d * row_vecs;
    for (uint32_t i = threadIdx.x; i < row_vecs; i += blockDim.x)
        drow[i] = s >= 0 ? src[(size_t)s * row_vecs + i] : make_uint4(0, 0, 0, 0);
}

template <typename T> __device__ __forceinline__ float elem_f32(uint16_t bits);
template <> __device__ __forceinline__ float elem_f32<f16_t>(uint16_t bits) { return __half2float(__ushort_as_half(bits)); }
template <> __device__ __forceinline__ float elem_f32<bf16_t>(uint16_t bits) { return __uint_as_float((uint32_t)bits << 16); }

// Order of the argmax: a non-NaN value maps to an integer key that sorts like the value (-0 and +0 share
// a key, as they compare equal), NaN to the smallest integer, which never beats the starting key.
constexpr int kNoKey = (int)0x80000000;
constexpr uint32_t kNoIndex = 0xFFFFFFFFu; // "nothing seen": loses every tie
__device__ __forceinline__ int order_key(float v) {
    int b = __float_as_int(v);
    if ((b & 0x7fffffff) > 0x7f800000) return kNoKey; // NaN
    if (b == kNoKey) b = 0;                           // -0
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ bool better(int key, uint32_t i, int bkey, uint32_t bi) {
    return key > bkey || (key == bkey && i < bi);
}

// grid (batch), block 1024: 16-byte loads where the row start allows it, scalar head and tail.  The scan is
// bound by vector instructions, not by memory, when every element is compared on its own (seven
// instructions each); so a lane takes the maximum of the eight values of a load first (v_max3, NaN operands
// drop out), compares once per load, remembers only which load held its best value, and fetches that one load
// again at the end to find the element.
template <typename T>
__global__ __launch_bounds__(1024) void batch_find_max_kernel(uint32_t* __restrict__ out, const uint16_t* __restrict__ in,
                                                               uint32_t length) {
    __shared__ int s_key[16];
    __shared__ uint32_t s_idx[16];
    const uint16_t* row = in + (size_t)blockIdx.x * length;
    // elements before the first 16-byte boundary of the row, then whole vectors, then the tail
    const uint32_t head = min(length, (uint32_t)(((16 - ((uintptr_t)row & 15)) & 15) / 2));
    const uint32_t nvec = (length - head) / 8;
    const uint4* vrow = reinterpret_cast<const uint4*>(row + head);
    int best = kNoKey;
    uint32_t best_vec = kNoIndex;
    auto take = [&](const uint4& w, uint32_t k) { // k ascends within a lane: the first of equal maxima stays
        const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
        float m = elem_f32<T>((uint16_t)ws[0]);
#pragma unroll
        for (int e = 1; e < 8; ++e) m = fmaxf(m, elem_f32<T>((uint16_t)(ws[e >> 1] >> (16 * (e & 1))))); // NaN only if all are
        const int key = order_key(m);
        if (key > best) { best = key; best_vec = k; }
    };
    // One workgroup (one CU) per row: what a CU streams is bounded by the bytes it has in flight, so every lane
    // keeps eight 16-byte loads outstanding (128 KiB per CU).
    uint32_t k = threadIdx.x;
    const uint32_t nt = blockDim.x;
    for (; k < nvec; k += 8 * nt) { // (the last pass re-reads the row's last load where it runs past the end)
        uint4 w[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) w[u] = vrow[min(k + u * nt, nvec - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (k + u * nt < nvec) take(w[u], k + u * nt);
    }
    uint32_t best_i = kNoIndex;
    if (best_vec != kNoIndex) { // the first element of that load with the lane's best key
        const uint4 w = vrow[best_vec];
        const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int e = 7; e >= 0; --e)
            if (order_key(elem_f32<T>((uint16_t)(ws[e >> 1] >> (16 * (e & 1))))) == best) best_i = head + 8 * best_vec + e;
    }
    auto take_one = [&](uint32_t i) {
        const int key = order_key(elem_f32<T>(row[i]));
        if (key != kNoKey && better(key, i, best, best_i)) { best = key; best_i = i; }
    };
    for (uint32_t i = threadIdx.x; i < head; i += blockDim.x) take_one(i);
    for (uint32_t i = head + 8 * nvec + threadIdx.x; i < length; i += blockDim.x) take_one(i);
    // wave64 reduction, then one value per wave through LDS
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const int ok = __shfl_xor(best, off, 64);
        const uint32_t oi = __shfl_xor(best_i, off, 64);
        if (better(ok, oi, best, best_i)) { best = ok; best_i = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { s_key[wave] = best; s_idx[wave] = best_i; }
    __syncthreads();
    if (wave == 0) {
        const int nw = blockDim.x >> 6;
        best = lane < nw ? s_key[lane] : kNoKey;
        best_i = lane < nw ? s_idx[lane] : kNoIndex;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) {
            const int ok = __shfl_xor(best, off, 64);
            const uint32_t oi = __shfl_xor(best_i, off, 64);
            if (better(ok, oi, best, best_i)) { best = ok; best_i = oi; }
        }
        if (lane == 0) out[blockIdx.x] = best_i == kNoIndex ? 0u : best_i; // no non-NaN element: 0
    }
}

static int check_rows(const void* a, const void* b, int dtype, uint32_t hidden) {
    if (!a || !b) return BZ_ERR_BAD_ARG;
    if (dtype != BZ_F16 && dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED;
    if (hidden == 0 || hidden % 8) return BZ_ERR_UNSUPPORTED;
    if (((uintptr_t)a | (uintptr_t)b) % 16) return BZ_ERR_BAD_ARG;
    return 0;
}

} // namespace bz

using namespace bz;

extern "C" int bz_embedding(void* output, const uint32_t* token_ids, const int32_t* out_loc, const void* weight,
                            int dtype, uint32_t num_tokens, uint32_t hidden_size, void* stream) {
    if (int rc = check_rows(output, weight, dtype, hidden_size)) return rc;
    if (!token_ids) return BZ_ERR_BAD_ARG;
    if (num_tokens == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream, (uint4*)output,
                       (const uint4*)weight, token_ids, out_loc, (const int32_t*)nullptr, hidden_size / 8);
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_gather_last_token(void* output, const void* tokens, const int32_t* ragged_indptr, int dtype,
                                    uint32_t num_tokens, uint32_t batch_size, uint32_t hidden_size, void* stream) {
    (void)num_tokens;
    if (int rc = check_rows(output, tokens, dtype, hidden_size)) return rc;
    if (!ragged_indptr) return BZ_ERR_BAD_ARG;
    if (batch_size == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(batch_size), dim3(256), 0, (hipStream_t)stream, (uint4*)output,
                       (const uint4*)tokens, (const uint32_t*)nullptr, (const int32_t*)nullptr, ragged_indptr,
                       hidden_size / 8);
    BZ_LAUNCH_CHECK();
    return 0;
}

extern "C" int bz_batch_find_max(uint32_t* output_indices, const void* input, int dtype, uint32_t batch_size,
                                 uint32_t length, void* stream) {
    if (!output_indices || !input) return BZ_ERR_BAD_ARG;
    if (dtype != BZ_F16 && dtype != BZ_BF16) return BZ_ERR_UNSUPPORTED;
    if (length == 0) return BZ_ERR_BAD_ARG;
    if ((uintptr_t)input % 2) return BZ_ERR_BAD_ARG;
    if (batch_size == 0) return 0;
    if (dtype == BZ_F16)
        hipLaunchKernelGGL(batch_find_max_kernel<f16_t>, dim3(batch_size), dim3(1024), 0, (hipStream_t)stream,
                           output_indices, (const uint16_t*)input, length);
    else
        hipLaunchKernelGGL(batch_find_max_kernel<bf16_t>, dim3(batch_size), dim3(1024), 0, (hipStream_t)stream,
                           output_indices, (const uint16_t*)input, length);
    BZ_LAUNCH_CHECK();
    return 0;
}
