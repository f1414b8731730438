// hipBLASLt implementation of the layers' GEMM boundary: replaces util::CublasWrapper::gemm
// (src/util/cublas_wrapper.h:183-207).  Row-major C[m,n] = A[m,k] B[k,n] is issued as the column-major
// product C^T[n,m] = B^T[n,k] A^T[k,m] with no transposes, the same operand swap the reference uses.
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

    void gemm(int m, int n, int k, const void* A, const void* B, void* C) override {
        Plan& p = plan(m, n, k);
        const float alpha = 1.f, beta = 0.f;
        // column-major view: D[n,m] = B[n,k] * A[k,m]
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
    // descriptors and the heuristic's first choice are kept per shape: a layer calls four shapes per step
    Plan& plan(int m, int n, int k) {
        const auto key = std::make_tuple(m, n, k);
        auto it = plans_.find(key);
        if (it != plans_.end()) return it->second;
        Plan p;
        check(hipblasLtMatmulDescCreate(&p.op, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
        check(hipblasLtMatrixLayoutCreate(&p.a, dtype_, (uint64_t)n, (uint64_t)k, (int64_t)n), "layout B^T");
        check(hipblasLtMatrixLayoutCreate(&p.b, dtype_, (uint64_t)k, (uint64_t)m, (int64_t)k), "layout A^T");
        check(hipblasLtMatrixLayoutCreate(&p.c, dtype_, (uint64_t)n, (uint64_t)m, (int64_t)n), "layout C^T");
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
    std::map<std::tuple<int, int, int>, Plan> plans_;
};

} // namespace blitz::util
