// The dense-GEMM boundary of the layers.  The reference calls util::CublasWrapper::gemm
// (src/util/cublas_wrapper.h:183-207, row-major C[m,n] = A[m,k] B[k,n]); dense GEMM is outside this
// library, so the layers take any implementation of this interface (hipBLASLt in an engine).
#pragma once

namespace blitz::util {

class GemmWrapper {
  public:
    virtual ~GemmWrapper() = default;
    /// row-major, no transposes: C[m, n] = A[m, k] * B[k, n], all device pointers of the layer's DType
    virtual void gemm(int m, int n, int k, const void* A, const void* B, void* C) = 0;
};

} // namespace blitz::util
