// Gated-linear-unit block of one transformer layer: the call-site contract of src/layer/glu.h.
#pragma once

#include <algorithm>
#include <cstdint>
#include <functional>

#include "../kernel/activation.h"
#include "../kernel/add.h"
#include "../kernel/rms_norm.h"
#include "../util/gemm_wrapper.h"

namespace blitz::layer {

template<typename DType>
class GatedLinearUnit {
  public:
    using AllReduce = std::function<void(DType*, size_t)>;

    /// weights from *seg_iter: post-attention norm [h] | gate_up [h, 2*I/tp] (each row gate then up,
    /// src/layer/glu.h:70-74) | down [I/tp, h]
    GatedLinearUnit(util::GemmWrapper* gemm, uint32_t hidden, uint32_t inter, DType* workspace_ptr, DType** seg_iter,
                    uint32_t tp_size = 1, AllReduce all_reduce = nullptr) :
        gemm_(gemm), all_reduce_(std::move(all_reduce)), hidden_(hidden), inter_(inter / tp_size), tp_(tp_size),
        workspace_(workspace_ptr) {
        norm_w_ = *seg_iter;
        gate_up_w_ = norm_w_ + hidden_;
        down_w_ = gate_up_w_ + 2 * (size_t)hidden_ * inter_;
        *seg_iter = down_w_ + (size_t)hidden_ * inter_;
    }

    size_t size_in_bytes() const { return ((size_t)hidden_ + 3 * (size_t)hidden_ * inter_) * sizeof(DType); }

    /// src/layer/glu.h:86-96.  Planes: [residual N*h][input = gate_up_state N*max(h,I)][gate_up_proj = down_proj].
    void forward(const uint32_t num_tokens, DType* buf = nullptr) {
        const size_t N = num_tokens;
        DType* residual = buf ? buf : workspace_;
        DType* input = workspace_ + N * hidden_;
        DType* gate_up_proj = input + N * std::max(hidden_, inter_);
        DType* gate_up_state = input;
        DType* down_proj = gate_up_proj;

        using util::GemmOp;
        kernel::add_rms_norm(input, residual, norm_w_, num_tokens, hidden_, 1e-5f, stream_);
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)(2 * inter_), (int)hidden_, input, gate_up_w_, gate_up_proj);
        kernel::silu_and_mul(gate_up_proj, gate_up_state, num_tokens, inter_, stream_);
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)hidden_, (int)inter_, gate_up_state, down_w_, down_proj);
        if (tp_ > 1 && all_reduce_) all_reduce_(down_proj, N * hidden_);
        kernel::add_residual(down_proj, residual, num_tokens, hidden_, stream_);
    }

    /// stream of this block's element-wise kernels (default: the process-wide option); the GEMM wrapper has its own
    void set_stream(void* stream) { stream_ = stream; }

  private:
    util::GemmWrapper* gemm_;
    AllReduce all_reduce_;
    const uint32_t hidden_, inter_, tp_;
    DType* workspace_;
    void* stream_ = kernel::kStreamFromOptions;
    DType *norm_w_, *gate_up_w_, *down_w_;
};

} // namespace blitz::layer
