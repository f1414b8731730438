// hipBLASLt implementation of the layers' GEMM boundary: replaces util::CublasWrapper
// (src/util/cublas_wrapper.h:144-207).  A row-major product C = op(A) op(B) is issued as the column-major
// product C^T = op(B)^T op(A)^T with the operands swapped and their transpose flags kept, the same trick
// the reference plays on cuBLAS (cublas_wrapper.h:183-207); batches map to hipBLASLt's strided batches.
// Accumulation is fp32 (the reference asks cuBLAS for fp16 accumulation, cublas_wrapper.h:144-146; the
// matrix cores of gfx950 accumulate in fp32 at full rate, so nothing is gained by narrowing it).
// Plain library GEMM: this header only drives hipBLASLt and links -lhipblaslt; libbz_hip.so does not
// depend on it.
#pragma once

#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <tuple>

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include "gemm_wrapper.h"

namespace blitz::util {

class HipblasLtGemm : public GemmWrapper {
  public:
    /// dtype: HIP_R_16F or HIP_R_16BF (the layer's DType); workspace is allocated once, here
    explicit HipblasLtGemm(hipDataType dtype, hipStream_t stream = nullptr, size_t workspace_bytes = 32u << 20)
        : dtype_(dtype), stream_(stream), workspace_bytes_(workspace_bytes) {
        check(hipblasLtCreate(&handle_), "hipblasLtCreate");
        if (hipMalloc(&workspace_, workspace_bytes_) != hipSuccess) throw std::runtime_error("HipblasLtGemm: workspace");
        check(hipblasLtMatmulPreferenceCreate(&pref_), "hipblasLtMatmulPreferenceCreate");
        check(hipblasLtMatmulPreferenceSetAttribute(pref_, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes_,
                                                    sizeof(workspace_bytes_)),
              "hipblasLtMatmulPreferenceSetAttribute");
    }
    ~HipblasLtGemm() override {
        for (auto& kv : plans_) {
            hipblasLtMatmulDescDestroy(kv.second.op);
            hipblasLtMatrixLayoutDestroy(kv.second.a);
            hipblasLtMatrixLayoutDestroy(kv.second.b);
            hipblasLtMatrixLayoutDestroy(kv.second.c);
        }
        hipblasLtMatmulPreferenceDestroy(pref_);
        (void)hipFree(workspace_);
        hipblasLtDestroy(handle_);
    }
    HipblasLtGemm(const HipblasLtGemm&) = delete;
    HipblasLtGemm& operator=(const HipblasLtGemm&) = delete;

    void set_stream(hipStream_t s) { stream_ = s; }

    using GemmWrapper::gemm;
    using GemmWrapper::gemmBatched;
    using GemmWrapper::gemmStridedBatched;

    void gemmStridedBatched(GemmOp transa, GemmOp transb, int m, int n, int k, float alpha, const void* A,
                            long long int stride_a, const void* B, long long int stride_b, float beta, void* C,
                            long long int stride_c, int batchCount) override {
        if (m <= 0 || n <= 0 || k <= 0 || batchCount <= 0) return;
        Plan& p = plan(transa, transb, m, n, k, stride_a, stride_b, stride_c, batchCount);
        // column-major view: C^T[n,m] = op(B)^T[n,k] * op(A)^T[k,m]
        check(hipblasLtMatmul(handle_, p.op, &alpha, B, p.a, A, p.b, &beta, C, p.c, C, p.c, &p.algo, workspace_,
                              workspace_bytes_, stream_),
              "hipblasLtMatmul");
    }

  private:
    struct Plan {
        hipblasLtMatmulDesc_t op;
        hipblasLtMatrixLayout_t a, b, c;
        hipblasLtMatmulAlgo_t algo;
    };
    typedef std::tuple<int, int, int, int, int, long long, long long, long long, int> Key;
    static void set_batch(hipblasLtMatrixLayout_t l, int batch, long long stride) {
        const int32_t bc = batch;
        const int64_t st = stride;
        check(hipblasLtMatrixLayoutSetAttribute(l, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &bc, sizeof(bc)), "batch count");
        check(hipblasLtMatrixLayoutSetAttribute(l, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &st, sizeof(st)),
              "batch stride");
    }
    // descriptors and the heuristic's first choice are kept per call shape: a layer calls four shapes per step
    Plan& plan(GemmOp transa, GemmOp transb, int m, int n, int k, long long sa, long long sb, long long sc, int batch) {
        const Key key = std::make_tuple((int)transa, (int)transb, m, n, k, sa, sb, sc, batch);
        auto it = plans_.find(key);
        if (it != plans_.end()) return it->second;
        Plan p;
        check(hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
        // the library's first operand is the caller's B, its second the caller's A, each with its own flag
        const hipblasOperation_t op_first = transb == GemmOp::N ? HIPBLAS_OP_N : HIPBLAS_OP_T;
        const hipblasOperation_t op_second = transa == GemmOp::N ? HIPBLAS_OP_N : HIPBLAS_OP_T;
        check(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSA, &op_first, sizeof(op_first)), "transa");
        check(hipblasLtMatmulDescSetAttribute(p.op, HIPBLASLT_MATMUL_DESC_TRANSB, &op_second, sizeof(op_second)), "transb");
        // stored shapes in column-major terms: B row-major [k,n] is n x k (ld n); transposed storage [n,k] is k x n (ld k)
        if (transb == GemmOp::N) check(hipblasLtMatrixLayoutCreate(&p.a, dtype_, (uint64_t)n, (uint64_t)k, (int64_t)n), "layout B");
        else check(hipblasLtMatrixLayoutCreate(&p.a, dtype_, (uint64_t)k, (uint64_t)n, (int64_t)k), "layout B");
        if (transa == GemmOp::N) check(hipblasLtMatrixLayoutCreate(&p.b, dtype_, (uint64_t)k, (uint64_t)m, (int64_t)k), "layout A");
        else check(hipblasLtMatrixLayoutCreate(&p.b, dtype_, (uint64_t)m, (uint64_t)k, (int64_t)m), "layout A");
        check(hipblasLtMatrixLayoutCreate(&p.c, dtype_, (uint64_t)n, (uint64_t)m, (int64_t)n), "layout C");
        if (batch > 1) {
            set_batch(p.a, batch, sb);
            set_batch(p.b, batch, sa);
            set_batch(p.c, batch, sc);
        }
        hipblasLtMatmulHeuristicResult_t res[1];
        int found = 0;
        check(hipblasLtMatmulAlgoGetHeuristic(handle_, p.op, p.a, p.b, p.c, p.c, pref_, 1, res, &found),
              "hipblasLtMatmulAlgoGetHeuristic");
        if (found < 1) throw std::runtime_error("HipblasLtGemm: no algorithm for this shape");
        p.algo = res[0].algo;
        return plans_.emplace(key, p).first->second;
    }
    static void check(hipblasStatus_t s, const char* what) {
        if (s != HIPBLAS_STATUS_SUCCESS)
            throw std::runtime_error(std::string("HipblasLtGemm: ") + what + " failed with status " + std::to_string((int)s));
    }

    hipDataType dtype_;
    hipStream_t stream_;
    uint64_t workspace_bytes_;
    void* workspace_ = nullptr;
    hipblasLtHandle_t handle_ = nullptr;
    hipblasLtMatmulPreference_t pref_ = nullptr;
    std::map<Key, Plan> plans_;
};

} // namespace blitz::util
