// The dense-GEMM boundary of the layers: the call shapes of util::CublasWrapper
// (src/util/cublas_wrapper.h:71-131) -- gemm, gemmBatched and gemmStridedBatched with and without
// alpha/beta, row-major operands, a transpose flag per input -- over any backend.  Dense GEMM is outside
// libbz_hip.so, so the layers take an implementation of this interface (hipBLASLt in an engine:
// hipblaslt_gemm.h).
//
// Row-major semantics, as the reference documents them (cublas_wrapper.h:33-68):
//   C[b] (m x n, leading dimension n) = alpha * op(A[b]) * op(B[b]) + beta * C[b]
//   A[b] is stored m x k (ld k) when transa == GemmOp::N, k x m (ld m) when GemmOp::T;
//   B[b] is stored k x n (ld n) when transb == GemmOp::N, n x k (ld k) when GemmOp::T;
//   matrix b of an operand starts stride_{a,b,c} elements after matrix b-1.
#pragma once

namespace blitz::util {

enum class GemmOp { N, T }; // stands where the reference passes CUBLAS_OP_N / CUBLAS_OP_T

class GemmWrapper {
  public:
    virtual ~GemmWrapper() = default;

    /// src/util/cublas_wrapper.h:71-88: the one form every other reduces to.  Device pointers of the
    /// layer's element type; alpha and beta are applied in fp32.
    virtual void gemmStridedBatched(GemmOp transa, GemmOp transb, int m, int n, int k, float alpha, const void* Aarray,
                                    long long int stride_a, const void* Barray, long long int stride_b, float beta,
                                    void* Carray, long long int stride_c, int batchCount) = 0;

    /// src/util/cublas_wrapper.h:94-108: alpha = 1, beta = 0
    void gemmStridedBatched(GemmOp transa, GemmOp transb, int m, int n, int k, const void* Aarray,
                            long long int stride_a, const void* Barray, long long int stride_b, void* Carray,
                            long long int stride_c, int batchCount) {
        gemmStridedBatched(transa, transb, m, n, k, 1.0f, Aarray, stride_a, Barray, stride_b, 0.0f, Carray, stride_c,
                           batchCount);
    }
    /// src/util/cublas_wrapper.h:115-126: matrices stored back to back
    void gemmBatched(GemmOp transa, GemmOp transb, int m, int n, int k, const void* Aarray, const void* Barray,
                     void* Carray, int batchCount) {
        gemmStridedBatched(transa, transb, m, n, k, Aarray, (long long)m * k, Barray, (long long)k * n, Carray,
                           (long long)m * n, batchCount);
    }
    /// src/util/cublas_wrapper.h:132-142, as called at src/layer/attn.h:139-171,206-215 and glu.h:109-136
    void gemm(GemmOp transa, GemmOp transb, int m, int n, int k, const void* Aarray, const void* Barray, void* Carray) {
        gemmBatched(transa, transb, m, n, k, Aarray, Barray, Carray, 1);
    }
};

} // namespace blitz::util
