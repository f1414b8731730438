// Attention block of one transformer layer: the call-site contract of src/layer/attn.h of the
// BlitzScale worker (same constructor roles, same forward() signature and workspace planes), with the
// attention-side work routed to the gfx950 kernels:
//   decode : the one-call decode step (paged batch decode over the cached tokens, then a kernel that rotates
//            and appends the new K/V rows, adds the new token's term and folds the split-K partials)
//   prefill: KV page store with K rotated on the way (into the pages and in place), then ragged causal
//            attention that rotates q in registers
// K is cached rotated, so no kernel ever rotates cached K again.
#pragma once

#include <cstdint>
#include <functional>

#include "../kernel/attention.h"
#include "../kernel/flashinfer_types.h"
#include "../kernel/page.h"
#include "../kernel/rms_norm.h"
#include "../util/gemm_wrapper.h"

namespace blitz::layer {

template<typename DType, typename IdType>
class Attention {
  public:
    using AllReduce = std::function<void(DType*, size_t)>; // in-place sum over the TP group (src/layer/attn.h:217-233)

    /// weights are laid out back to back from *seg_iter as in the reference (src/layer/attn.h:85-91):
    /// input norm [h] | Wq [h, Hq*D/tp] | Wk [h, Hkv*D/tp] | Wv | Wo [Hq*D/tp, h]
    Attention(util::GemmWrapper* gemm, kernel::BatchPrefillRaggedHandler<DType, IdType>* prefill_handle,
              kernel::BlitzBatchDecodeHandler<DType, IdType>* decode_handle, uint32_t head_dim, uint32_t hidden_dim,
              uint32_t num_qo_head, uint32_t num_kv_head, DType* workspace_ptr, DType** seg_iter, uint32_t tp_size = 1,
              AllReduce all_reduce = nullptr) :
        gemm_(gemm), prefill_(prefill_handle), decode_(decode_handle), all_reduce_(std::move(all_reduce)),
        Hq_(num_qo_head / tp_size), Hkv_(num_kv_head / tp_size), D_(head_dim), hidden_(hidden_dim), tp_(tp_size),
        workspace_(workspace_ptr) {
        norm_w_ = *seg_iter;
        wq_ = norm_w_ + hidden_;
        wk_ = wq_ + (size_t)Hq_ * D_ * hidden_;
        wv_ = wk_ + (size_t)Hkv_ * D_ * hidden_;
        wo_ = wv_ + (size_t)Hkv_ * D_ * hidden_;
        *seg_iter = wo_ + (size_t)Hq_ * D_ * hidden_;
    }

    size_t size_in_bytes() const noexcept {
        return ((size_t)hidden_ + 2 * (size_t)Hq_ * D_ * hidden_ + 2 * (size_t)Hkv_ * D_ * hidden_) * sizeof(DType);
    }

    /// src/layer/attn.h:98-103.  qo_indptr_d != nullptr selects prefill; buf replaces the residual plane.
    /// Workspace planes: [residual N*h][input N*h][q N*Hq*D | k N*Hkv*D | v N*Hkv*D][attn_state N*Hq*D];
    /// the O projection lands in the input plane (src/layer/attn.h:104-115).
    void forward(const uint32_t num_tokens, IdType* qo_indptr_d, kernel::PageTable<DType, IdType>& page_table,
                 DType* buf = nullptr) {
        const size_t N = num_tokens;
        DType* residual = buf ? buf : workspace_;
        DType* input = workspace_ + N * hidden_;
        DType* q = input + N * hidden_;
        DType* k = q + N * Hq_ * D_;
        DType* v = k + N * Hkv_ * D_;
        DType* attn_state = v + N * Hkv_ * D_;
        DType* o_proj = input;

        // stream and RoPE base travel with the handlers (one set per model); the page writes are handed the same
        // handler's options, whatever the table points at, so pages and attention cannot disagree
        void* stream = (qo_indptr_d ? prefill_->options : decode_->options).stream;
        kernel::rms_norm(residual, norm_w_, input, num_tokens, hidden_, 1e-5f, stream);
        // Three projections into three planes.  (The reference batches them into one or two row-major
        // GEMMs, src/layer/attn.h:137-171, whose output would interleave q, k and v per token while the
        // attention kernels read separate planes; the planes are what the kernel contract needs.)
        using util::GemmOp;
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)(Hq_ * D_), (int)hidden_, input, wq_, q);
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)(Hkv_ * D_), (int)hidden_, input, wk_, k);
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)(Hkv_ * D_), (int)hidden_, input, wv_, v);
        if (qo_indptr_d) {
            // K rotated once, into the pages and in place, while the pages are written; q is rotated in registers
            // inside the attention kernel (read once, never written)
            kernel::store_prefill_kv_cache(page_table, k, v, qo_indptr_d, num_tokens, static_cast<DType*>(nullptr), 0,
                                           nullptr, nullptr, /*rotate=*/2, &prefill_->options);
            kernel::batch_prefill_attention(*prefill_, q, qo_indptr_d, k, v, qo_indptr_d, attn_state,
                                            page_table.batch_size, Hq_, Hkv_, D_, BZ_ROPE_Q_ONLY);
        } else {
            // append (new K rotated on its way in) + decode (q rotated inside the kernels) as one call
            kernel::decode_attention_step(*decode_, q, k, v, page_table, attn_state, Hq_);
        }
        gemm_->gemm(GemmOp::N, GemmOp::N, (int)N, (int)hidden_, (int)(Hq_ * D_), attn_state, wo_, o_proj);
        if (tp_ > 1 && all_reduce_) all_reduce_(o_proj, N * hidden_);
    }

  private:
    util::GemmWrapper* gemm_;
    kernel::BatchPrefillRaggedHandler<DType, IdType>* prefill_;
    kernel::BlitzBatchDecodeHandler<DType, IdType>* decode_;
    AllReduce all_reduce_;
    const uint32_t Hq_, Hkv_, D_, hidden_, tp_;
    DType* workspace_;
    DType *norm_w_, *wq_, *wk_, *wv_, *wo_;
};

} // namespace blitz::layer
