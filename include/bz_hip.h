/*
 * bz_hip.h -- C ABI of the MI355X (gfx950) paged-attention compute path.
 *
 * Every entry point replaces one wrapper of the BlitzScale worker's src/kernel
 * directory (cited per function, paths relative to the reference checkout).
 * Conventions shared by all of them, following the reference wrappers:
 *   - all tensors, page tables and workspaces are caller-owned DEVICE memory
 *     unless a parameter name ends in _h (host memory);
 *   - launches are asynchronous on `stream` (a hipStream_t passed as void*;
 *     NULL = the legacy default stream the reference uses everywhere) and never
 *     synchronise the device;
 *   - the return value is 0 on success, otherwise a hipError_t value (the C++
 *     shim turns it into std::runtime_error like the reference does with
 *     cudaError_t) or one of the BZ_ERR_* codes below for argument errors;
 *   - nothing here allocates device memory except bz_kv_pool_alloc.
 */
#ifndef BZ_HIP_H_
#define BZ_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types */
#define BZ_F16 0
#define BZ_BF16 1
#define BZ_E4M3 2 /* OCP e4m3fn, KV pool only */
#define BZ_F32 3  /* attention output only (test instantiation) */

/* RoPE handling inside the attention kernels (Llama rotate-half, f_i = theta^(-2i/D)) */
#define BZ_ROPE_NONE 0   /* q and cached K are used as they are                       */
#define BZ_ROPE_Q_ONLY 1 /* q rotated at position seq_len-1; cached K already rotated */
#define BZ_ROPE_FULL 2   /* q rotated at seq_len-1 and every cached K at its own      */
                         /* position: the reference's kRoPELlama with a raw-K cache   */

/* argument errors (outside the hipError_t range) */
#define BZ_ERR_BAD_ARG 10001
#define BZ_ERR_UNSUPPORTED 10002
#define BZ_ERR_WORKSPACE 10003
#define BZ_ERR_NOT_PLANNED 10004
#define BZ_ERR_NO_PAGES 10005 /* page allocator exhausted, or a page table outgrew its pinned chunk */

/* In-page element order of the KV pool. */
#define BZ_LAYOUT_NHD 0 /* [page][K|V][slot][head][dim]: the reference's (page.h:24-32) */
#define BZ_LAYOUT_HND 1 /* [page][K|V][head][slot][dim]: one (page, head) tile contiguous */

/*
 * One layer plane of the paged KV pool plus the per-batch CSR page table: the plain-C
 * image of blitz::kernel::PageTable (src/kernel/page.h:12-64).  Element address relative
 * to k_data / v_data:  page*stride_page + slot*stride_n + head*stride_h + d   (elements).
 * seq_len_b = (indptr[b+1]-indptr[b]-1)*page_size + last_page_len[b]   (page.cu:38-40).
 *
 * steps_ahead (optional, no counterpart in the reference): a device int32.  When non-NULL the table
 * describes the batch steps_ahead[0] decode steps in the FUTURE: every sequence is at present that many
 * tokens shorter than indptr / last_page_len say, and the pages of the tokens to come are already in
 * `indices`.  bz_append_decode_kv and bz_batch_decode then work at the present length
 * (seq_len_b - steps_ahead[0]; a sequence this leaves without tokens is skipped / yields a zero row).
 * A host that grows the table H steps ahead uploads it and plans ONCE, sets the counter to H-1, and runs
 * H decode steps (bz_steps_ahead_advance after each) without touching table, plan or counter from the
 * host again: the per-step plan() and table upload of src/model/llama.h:363-375 and
 * src/blitz/stub.h:1288-1313 leave the step, and a whole step can be replayed from one HIP graph.
 * The prefill store ignores it.
 */
typedef struct bz_paged_kv {
    void* k_data;
    void* v_data;
    const int32_t* indices;       /* [indptr[batch_size]] page ids */
    const int32_t* indptr;        /* [batch_size + 1]               */
    const int32_t* last_page_len; /* [batch_size], 1..page_size     */
    uint32_t batch_size;
    uint32_t page_size;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    uint64_t stride_page;
    uint64_t stride_n;
    uint64_t stride_h;
    int32_t kv_dtype;             /* BZ_F16 | BZ_BF16 | BZ_E4M3 */
    int32_t reserved;
    const int32_t* steps_ahead;   /* optional device scalar, see above; NULL = the table is the present */
} bz_paged_kv_t;

/* Fill the stride fields for a layout (stride_page = 2*H*P*D for both; page.h:59-61). */
void bz_paged_kv_set_layout(bz_paged_kv_t* kv, int layout);

/* Bytes of one layer plane / of the whole pool: 2*L*max_pages*Hkv*P*D elements
 * (src/blitz/cache_manager.h:136-142).  Address arithmetic is 64-bit throughout. */
uint64_t bz_kv_pool_bytes(uint32_t num_layers, uint64_t max_pages, uint32_t num_kv_heads, uint32_t page_size,
                          uint32_t head_dim, int kv_dtype);
/* hipMalloc of the pool (replaces the cudaMalloc at cache_manager.h:136-142). */
int bz_kv_pool_alloc(void** base, uint64_t bytes);
int bz_kv_pool_free(void* base);
/* k_data / v_data of layer `layer` (the pointer bump of src/model/llama.h:356-359,378-381). */
void bz_kv_layer_view(bz_paged_kv_t* kv, void* pool_base, uint32_t layer, uint64_t max_pages);

/* ---------------------------------------------------------------------------------------
 * Decode plan: replaces BlitzBatchDecodeHandler::plan (src/kernel/flashinfer_types.h:44-72,
 * flashinfer_types.cu:52-80).  Host-side scheduling from the HOST copies of indptr and
 * last_page_len: cuts every sequence into page-aligned segments (split-K), balances them
 * over the compute units and copies the schedule into int_buffer (device).  float_buffer
 * (device) receives the split-K partial results at run time.  Synchronous host work plus
 * one async H2D copy on `stream`, like the reference's plan().
 * split_tokens: contexts longer than this are always split (0 = library default 2048,
 * UINT32_MAX = never split: one piece per sequence).
 * ------------------------------------------------------------------------------------- */
typedef struct bz_decode_plan bz_decode_plan_t;

bz_decode_plan_t* bz_decode_plan_create(void); /* create_flashinfer_decode_handler, flashinfer_types.cu:18-22 */
void bz_decode_plan_destroy(bz_decode_plan_t* plan);
int bz_decode_plan(bz_decode_plan_t* plan, void* float_buffer, size_t float_buffer_bytes, void* int_buffer,
                   size_t int_buffer_bytes, const int32_t* indptr_h, const int32_t* last_page_len_h,
                   uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim,
                   uint32_t page_size, uint32_t split_tokens, void* stream);
/* Workspace sizing (no counterpart in the reference, which fixes 128 MiB + 8 MiB, src/model/llama.h:111-112):
 * runs the same host-side scheduling and reports how many bytes of the two workspaces bz_decode_plan would
 * use for this batch with the matrix-core kernel where the shape allows it.  Touches no GPU when
 * num_compute_units is given (0 = ask the current device).  The handle must be planned again before the
 * next bz_batch_decode. */
int bz_decode_plan_workspace(bz_decode_plan_t* plan, const int32_t* indptr_h, const int32_t* last_page_len_h,
                             uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim,
                             uint32_t page_size, uint32_t split_tokens, uint32_t num_compute_units,
                             size_t* float_buffer_bytes, size_t* int_buffer_bytes);
/* The host copy of the last schedule built by bz_decode_plan / bz_decode_plan_workspace, for tests and
 * tools: records of ints_per_record int32 each, valid until the handle plans again.  which = 0: page-aligned
 * segments of the general kernel {seq, page_begin, page_end, partial | -1}; 1: its split sequences {seq,
 * first partial, count, 0}; 2: sequences without pages {seq}; 3: one record per 32-token tile of the
 * matrix-core kernel, in processing order {position in indices[] of the page of tokens 32t.., of tokens
 * 32t+16.., t, piece}; 4: wave-slot boundaries into those records; 5: pieces {seq, kv head, tile_begin,
 * tile_end, partial | -1, combine index | -1, partials of its (seq, kv head), first of them, indptr[seq],
 * pages, tokens, ...}; 6: split (seq, kv head)s {seq, kv head, first partial, count}; 7: every (seq with
 * pages, kv head) with its run of pieces {seq, kv head, first piece, count, indptr[seq], tokens, ...} (read by
 * bz_decode_step). */
int bz_decode_plan_host_schedule(const bz_decode_plan_t* plan, int which, const int32_t** data, size_t* num_records,
                                 uint32_t* ints_per_record);
/* introspection for tests and the bench: number of segments / of sequences that were split */
int bz_decode_plan_info(const bz_decode_plan_t* plan, uint32_t* num_segments, uint32_t* num_split_seqs,
                        uint32_t* num_workgroups);
/* introspection: 1 when bz_decode_step on this plan runs its two-launch form, 0 when it runs the append and the
 * decode calls one after the other (see bz_decode_step); negative on error.  No counterpart in the reference. */
int bz_decode_plan_step_form(const bz_decode_plan_t* plan);

/* Profiling aid (no counterpart in the reference): when both handles are non-NULL hipEvent_t values,
 * the next bz_batch_decode calls on this plan record them on the launch stream immediately before
 * and after the decode kernel itself (the split-K combine launch that may follow is outside the
 * pair).  Pass NULL, NULL to switch it off. */
int bz_decode_plan_set_timing_events(bz_decode_plan_t* plan, void* start_event, void* stop_event);

/*
 * batch_decode_attention (src/kernel/attention.h:24-31, attention_decode.cu:13-40).
 * q, out: [batch, num_qo_heads, head_dim] of q_dtype (out_dtype may be BZ_F32 for tests).
 * sm_scale <= 0 selects 1/sqrt(head_dim) (the default the reference never overrides).
 * k_scale / v_scale: device fp32 [num_kv_heads] dequantisation factors for an e4m3 pool
 * (NULL = 1).  lse: optional device fp32 [batch, num_qo_heads] (reference passes nullptr).
 * BZ_ROPE_FULL (raw K in the cache, the reference's kRoPELlama): the first such call after a plan builds a table
 * of angles, 4 * head_dim bytes per position of the longest sequence, in the plan's float workspace behind the
 * split-K partials when there is room (it is only faster with it).
 */
int bz_batch_decode(bz_decode_plan_t* plan, const void* q, int q_dtype, const bz_paged_kv_t* kv, void* out,
                    int out_dtype, uint32_t num_qo_heads, int rope_mode, float rope_theta, float sm_scale,
                    const float* k_scale, const float* v_scale, float* lse, void* stream);

/*
 * One layer's decode-time attention step as ONE call: what append_decode_kv_cache followed by
 * batch_decode_attention compute (src/layer/attn.h:196-203), i.e. bz_append_decode_kv(kv, k_new, v_new, rope)
 * and then bz_batch_decode(q, rope ? BZ_ROPE_Q_ONLY : BZ_ROPE_NONE), in two launches instead of three and with
 * the append off the critical path: the decode kernel attends over every token but the newest (it does not
 * wait for the append), and a finishing kernel rotates and appends the new K/V rows, adds the new token's own
 * term from the caller's rows and folds the split-K partials.  q [B,Hq,D], k_new, v_new [B,Hkv,D] are read
 * only (q is rotated in registers); the pool receives the same bits bz_append_decode_kv writes; `out` agrees
 * with the two-call sequence to rounding (the summation order differs).  Needs a float workspace with room
 * for one partial per piece (bz_decode_plan_workspace reports it); where the matrix-core kernel does not
 * apply, or the workspace is too small, the call runs the two-call sequence itself.  It also does so where
 * that is the faster order: batches in which most (sequence, kv head)s fit one wave slot whole write their
 * final rows directly in the two calls, while the two-launch form would send each through a partial row
 * (bz_decode_plan_step_form tells which form a plan takes).  Launch only.
 */
int bz_decode_step(bz_decode_plan_t* plan, const void* q, int q_dtype, const void* k_new, const void* v_new,
                   const bz_paged_kv_t* kv, void* out, int out_dtype, uint32_t num_qo_heads, int rope,
                   float rope_theta, float sm_scale, const float* k_scale, const float* v_scale, float* lse,
                   void* stream);

/*
 * bz_batch_decode for callers that cannot allocate device memory or bring a float workspace along (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments, same kernels and bit-identical results as bz_batch_decode on the same plan,
 * except that the split-K partial results go to a fixed device array inside the library
 * (BZ_DECODE_NOALLOC_SCRATCH_BYTES per GPU, held from module load to process exit) instead of the float
 * workspace given to bz_decode_plan; that workspace is not touched by this call.  The call itself performs
 * no allocation, free, copy or synchronisation: it only launches kernels on `stream` (the array's address on
 * the current GPU is looked up by bz_decode_plan), so it may be recorded into a HIP graph.
 * Limit: the plan's partial results must fit the array (8256 bytes per partial of the matrix-core kernel,
 * 4*(head_dim+1)*num_qo_heads per partial of the general kernel; the rule is conservative: what either kernel
 * would need for this plan, whichever the call ends up running); otherwise BZ_ERR_WORKSPACE is returned
 * before anything is launched.  All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (two streams, two threads) race; calls in stream order are safe, and nothing in the array has to
 * be cleared between them (every partial the combine reads is written by the same call first).
 */
#define BZ_DECODE_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t bz_batch_decode_noalloc_scratch_bytes(void);
int bz_batch_decode_noalloc(bz_decode_plan_t* plan, const void* q, int q_dtype, const bz_paged_kv_t* kv, void* out,
                            int out_dtype, uint32_t num_qo_heads, int rope_mode, float rope_theta, float sm_scale,
                            const float* k_scale, const float* v_scale, float* lse, void* stream);

/* ---------------------------------------------------------------------------------------
 * Prefill plan: replaces BatchPrefillRaggedHandler::plan (flashinfer_types.h:12-41,
 * flashinfer_types.cu:24-49).  Builds the (request, q-tile) work list, longest first.
 * ------------------------------------------------------------------------------------- */
typedef struct bz_prefill_plan bz_prefill_plan_t;

bz_prefill_plan_t* bz_prefill_plan_create(void); /* create_flashinfer_prefill_handler, flashinfer_types.cu:12-16 */
void bz_prefill_plan_destroy(bz_prefill_plan_t* plan);
int bz_prefill_plan(bz_prefill_plan_t* plan, void* float_buffer, size_t float_buffer_bytes, void* int_buffer,
                    size_t int_buffer_bytes, const int32_t* qo_indptr_h, const int32_t* kv_indptr_h,
                    uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim,
                    uint32_t page_size, void* stream);

/* Host-only counterparts of bz_decode_plan_workspace / bz_decode_plan_host_schedule for the prefill plan:
 * the bytes of int_buffer the job list of this batch takes and the bytes of float_buffer that hold the angle
 * table of the in-register q rotation (512 per position of the longest request; optional, see
 * bz_batch_prefill_ragged), and the host copy of the list, one record of 8 ints per workgroup in launch order
 * {first q row of the request, q rows of the request (0 = padding entry), first q row of the tile inside the
 * request, q head, first K/V row of the request, K/V rows of the request, 0, 0}.  No GPU call. */
int bz_prefill_plan_workspace(bz_prefill_plan_t* plan, const int32_t* qo_indptr_h, const int32_t* kv_indptr_h,
                              uint32_t batch_size, uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim,
                              size_t* float_buffer_bytes, size_t* int_buffer_bytes);
int bz_prefill_plan_host_schedule(const bz_prefill_plan_t* plan, const int32_t** data, size_t* num_records,
                                  uint32_t* ints_per_record);

/* How bz_batch_prefill_ragged takes bf16 through its second contraction (no counterpart in the reference, whose
 * FlashInfer call rounds the probabilities to bf16's 8-bit significand; the stated tolerance does not allow that).
 * BZ_PREFILL_BF16_WIDEN_V (default): V tiles are widened to f16 on chip and the probabilities are f16 -- exact for
 * |v| in f16's range (2^-24 .. 65504; smaller values round to f16 subnormals or zero, larger ones become infinite).
 * BZ_PREFILL_BF16_HEAD_TAIL: V stays bf16 and the probabilities enter as head + tail of bf16 -- any range, two
 * matrix instructions per step.  A setting of the plan: it holds for every later call with it. */
#define BZ_PREFILL_BF16_WIDEN_V 0
#define BZ_PREFILL_BF16_HEAD_TAIL 1
int bz_prefill_plan_set_bf16_mode(bz_prefill_plan_t* plan, int mode);

/* Profiling aid, as bz_decode_plan_set_timing_events: two hipEvent_t handles recorded on the call's stream right
 * before and right after the launch of the attention kernel of bz_batch_prefill_ragged (not around the kernels that
 * rotate k or write the angle table in front of it).  Both NULL switches it off.  No counterpart in the reference. */
int bz_prefill_plan_set_timing_events(bz_prefill_plan_t* plan, void* start_event, void* stop_event);

/*
 * batch_prefill_attention (src/kernel/attention.h:9-22, attention_prefill.cu:11-46): ragged
 * attention, q [Nq,Hq,D], k,v [Nkv,Hkv,D], out [Nq,Hq,D].  The reference passes one array as qo_indptr and
 * kv_indptr (src/layer/attn.h:175-187): self-attention over each request.  With two arrays request b has
 * q rows for its LAST qo_len_b tokens only and K/V rows for all kv_len_b >= qo_len_b of them (a chunk of a
 * prompt attending to the whole prefix): q row i sits at position kv_len_b - qo_len_b + i.  causal != 0 masks
 * the K/V rows behind a q row's position.  The device arrays must hold what the plan was made from.
 * rope_mode BZ_ROPE_NONE: q, k used as they are.  BZ_ROPE_Q_ONLY: q rows are rotated by their position inside
 * the request in registers (q in memory stays as it is), k is expected rotated (bz_store_prefill_kv with
 * rope = 2 leaves it so).  BZ_ROPE_FULL, the reference's kRoPELlama: q as for BZ_ROPE_Q_ONLY, and the k rows
 * are rotated IN PLACE first (the caller's k buffer then holds rotated K for the page store that follows,
 * which must not rotate it again).  The angle table of the q rotation lives in the float workspace given to
 * bz_prefill_plan (512 bytes per position of the longest request; bz_prefill_plan_workspace reports it);
 * without room for it q is rotated in place by a separate launch instead.
 */
int bz_batch_prefill_ragged(bz_prefill_plan_t* plan, void* q, const int32_t* qo_indptr, void* k, void* v,
                            const int32_t* kv_indptr, void* out, int dtype, uint32_t batch_size,
                            uint32_t num_qo_heads, uint32_t num_kv_heads, uint32_t head_dim, int causal,
                            int rope_mode, float rope_theta, float sm_scale, void* stream);

/* ---------------------------------------------------------------------------------------
 * KV page writes
 * ------------------------------------------------------------------------------------- */
/* store_prefill_kv_cache (src/kernel/page.h:66-67, page.cu:21-94): token t of request b goes to
 * page indices[indptr[b]+t/P], slot t%P.  k, v: [N, Hkv, D] of src_dtype.
 * rope != 0 rotates K at position t on the way in.  rope == 2 also rotates the caller's k rows in place
 * (q is then left to bz_batch_prefill_ragged with BZ_ROPE_Q_ONLY, which rotates it in registers: the
 * fused RoPE of the prefill path).  With q_inout (optional, [N, Hq, D], num_qo_heads) given, q AND the
 * caller's k rows are rotated in place by the same angles, after which bz_batch_prefill_ragged runs
 * with BZ_ROPE_NONE.
 * k_scale / v_scale: device fp32 [Hkv]; for an e4m3 pool the value stored is quant(x / scale).
 * num_tokens: N, or BZ_NUM_TOKENS_FROM_INDPTR when the host does not know it (the reference's call has no
 * such argument and shapes its launch from page size and batch, page.cu:84-89).  Tokens of a request beyond
 * the pages its table row lists are dropped (the reference asserts seq_len >= append length, page.cu:43);
 * nothing is ever written outside the listed pages. */
#define BZ_NUM_TOKENS_FROM_INDPTR 0xFFFFFFFFu /* num_tokens: take ragged_indptr[batch_size], read on the device */
int bz_store_prefill_kv(const bz_paged_kv_t* kv, void* k, const void* v, int src_dtype,
                        const int32_t* ragged_indptr, uint32_t num_tokens, void* q_inout, uint32_t num_qo_heads,
                        int rope, float rope_theta, const float* k_scale, const float* v_scale, void* stream);

/* append_decode_kv_cache (src/kernel/page.h:69-70, page.cu:96-115): one new row per sequence at
 * position seq_len-1 (page indices[indptr[b+1]-1], slot last_page_len[b]-1).  k, v: [B, Hkv, D].
 * rope / q_inout as above with position seq_len-1: the fused RoPE + append of the decode path. */
int bz_append_decode_kv(const bz_paged_kv_t* kv, const void* k, const void* v, int src_dtype, void* q_inout,
                        uint32_t num_qo_heads, int rope, float rope_theta, const float* k_scale,
                        const float* v_scale, void* stream);

/* End of a decode step under a table that runs ahead (bz_paged_kv_t.steps_ahead): the counter goes down
 * by one, not below zero.  One tiny launch on `stream`, recordable into a HIP graph. */
int bz_steps_ahead_advance(int32_t* steps_ahead, void* stream);

/* Rotate (inverse == 0) or un-rotate (inverse != 0) the cached K rows of every sequence of the table in place, row t
 * of a sequence at position t: one pass at the speed of a copy.  The reference caches K as the projection left
 * it and rotates every cached row inside every decode call (kRoPELlama, src/kernel/attention_decode.cu:35); this
 * library caches K rotated and rotates q only.  A cache filled under the reference's convention (e.g. pages received
 * from a reference instance) is converted once with this call and then served by the fast decode path
 * (BZ_ROPE_Q_ONLY); inverse takes a cache back before it leaves for such a consumer.  Forward then inverse restores
 * the rows to within one rounding of the storage type.  f16 / bf16 pools, head_dim 64 or 128, page_size <= 128
 * (head_dim 128).  BZ_ROPE_FULL of bz_batch_decode remains for caches that must stay raw. */
int bz_rope_cached_k(const bz_paged_kv_t* kv, float rope_theta, int inverse, void* stream);

/* ---------------------------------------------------------------------------------------
 * element-wise kernels of src/layer's call sites
 * ------------------------------------------------------------------------------------- */
/* rms_norm (src/kernel/rms_norm.h:11-19, norm.cu:7-22); input may alias output (llama.h:389-391) */
int bz_rms_norm(const void* input, const void* weight, void* output, int dtype, uint32_t num_tokens,
                uint32_t hidden_size, float eps, void* stream);
/* add_rms_norm (rms_norm.h:26-34, norm.cu:24-39): residual += input; input = rms_norm(residual)*w */
int bz_add_rms_norm(void* input, void* residual, const void* weight, int dtype, uint32_t num_tokens,
                    uint32_t hidden_size, float eps, void* stream);
/* silu_and_mul (src/kernel/activation.h:7-16, activation.cu:9-26): input [N, 2I] gate first, output [N, I] */
int bz_silu_and_mul(const void* input, void* output, int dtype, uint32_t num_tokens, uint32_t inter_size,
                    void* stream);
/* add_residual (src/kernel/add.h:8-14, add.cu:13-61): residual += input, one rounding per element */
int bz_add_residual(const void* input, void* residual, int dtype, uint32_t num_tokens, uint32_t dim,
                    void* stream);

/* ---------------------------------------------------------------------------------------
 * row gathers and greedy sampling either side of the layer loop (src/model/llama.h)
 * ------------------------------------------------------------------------------------- */
/* embedding (src/kernel/embedding.h:7-36, embedding.cu:7-47): output[loc] = weight[token_ids[t]] for
 * t < num_tokens, rows of hidden_size 16-bit elements (hidden_size % 8 == 0); loc = t, or out_loc[t]
 * when out_loc is given (the tensor-parallel variant that scatters into a zeroed buffer). */
int bz_embedding(void* output, const uint32_t* token_ids, const int32_t* out_loc, const void* weight, int dtype,
                 uint32_t num_tokens, uint32_t hidden_size, void* stream);
/* gather_last_token (src/kernel/sampler.h:8-16, sampler.cu:7-54): output[b] = tokens[ragged_indptr[b+1]-1],
 * the whole row (the reference's kernel drops the lane offset on the destination, sampler.cu:21-24);
 * a request without tokens yields a zero row. */
int bz_gather_last_token(void* output, const void* tokens, const int32_t* ragged_indptr, int dtype,
                         uint32_t num_tokens, uint32_t batch_size, uint32_t hidden_size, void* stream);
/* batch_find_max (src/kernel/sampler.h:18-26, sampler.cu:80-135): output_indices[b] = argmax_i input[b][i]
 * over rows of `length` 16-bit elements: the smallest index of the largest non-NaN value, 0 for a row
 * that has none (the reference leaves ties to a race and the index undefined below -65400). */
int bz_batch_find_max(uint32_t* output_indices, const void* input, int dtype, uint32_t batch_size, uint32_t length,
                      void* stream);

/* ---------------------------------------------------------------------------------------
 * KV page wire format for migration between instances.  The reference sends one message of
 * stride_page elements per (page, layer) straight from the pool, request by request, prompt block by
 * prompt block, layer by layer (src/blitz/migration_manager.h:86-92 get_page_ptr, :455-467 send loop;
 * the receive loops mirror it).  bz_kv_pages_pack writes that byte stream into ONE contiguous device
 * buffer, so that one large transfer replaces the per-(page, layer) sends: chunk c = i*layer_cnt + l of
 * `wire` is page page_ids[i] of layer start_layer + l (stride_page elements, the page's in-pool
 * order).  bz_kv_pages_unpack scatters such a buffer to the receiver's own page ids.
 *   pool_base : layer 0 of a pool laid out [layer][page][...] with max_pages pages per layer
 *   kv        : geometry only (num_kv_heads, stride_page, stride_h, kv_dtype); its pointers are not read
 *   page_ids  : device array [num_pages], in the order the pages are to appear on the wire
 *   wire_dtype: the pool's type (bit copy), or BZ_E4M3 for a 16-bit pool: elements travel as
 *               e4m3(x / scale) and arrive as e4m3 * scale, scale = k_scale / v_scale[l*num_kv_heads +
 *               head] (device arrays [layer_cnt][num_kv_heads]; NULL = 1), half the bytes.
 * Page ids outside [0, max_pages) are skipped (pack writes zeros into their chunk of `wire`, unpack ignores
 * it).  Pages listed twice in an unpack race.  Launch only; no allocation, copy or synchronisation.
 * ------------------------------------------------------------------------------------- */
uint64_t bz_kv_wire_bytes(uint32_t num_pages, uint32_t layer_cnt, const bz_paged_kv_t* kv, int wire_dtype);
int bz_kv_pages_pack(const void* pool_base, uint64_t max_pages, const bz_paged_kv_t* kv, const int32_t* page_ids,
                     uint32_t num_pages, uint32_t start_layer, uint32_t layer_cnt, void* wire, int wire_dtype,
                     const float* k_scale, const float* v_scale, void* stream);
int bz_kv_pages_unpack(void* pool_base, uint64_t max_pages, const bz_paged_kv_t* kv, const int32_t* page_ids,
                       uint32_t num_pages, uint32_t start_layer, uint32_t layer_cnt, const void* wire,
                       int wire_dtype, const float* k_scale, const float* v_scale, void* stream);

/* ---------------------------------------------------------------------------------------
 * Host page-table logic: pool owner, first-fit page allocator and per-batch page tables in pinned
 * memory.  Replaces the integer semantics of src/blitz/cache_manager.h:123-324 and of the page-table
 * parts of src/blitz/batch.h (prefill constructor :206-276, update :280-295, filter :297-418,
 * extend :482-576).  Pure host work; with_device = 0 skips the pool and the pinned allocation so
 * that the logic can run without a GPU.  A batch's table is the blob [indices | indptr |
 * last_page_len] that Stub::forward uploads in one copy (src/blitz/stub.h:1288-1313).
 * ------------------------------------------------------------------------------------- */
typedef struct bz_cache_manager bz_cache_manager_t;

int bz_cm_create(bz_cache_manager_t** out, uint32_t num_kv_heads, uint32_t num_layers, uint32_t head_dim,
                 uint32_t page_size, uint32_t max_pages, int kv_dtype, int layout, int with_device);
void bz_cm_destroy(bz_cache_manager_t* cm);
/* new batch from prompt lengths: each prompt reserves len+1 slots (batch.h:246-250), lowest free page ids */
int bz_cm_batch_prefill(bz_cache_manager_t* cm, const int32_t* prompt_lens, uint32_t batch, int* batch_id);
/* every sequence grows by one slot, a full last page gets a new page (cache_manager.h:255-324) */
int bz_cm_batch_grow(bz_cache_manager_t* cm, int batch_id);
/* keep the listed sequences (ascending positions), free the pages of the others (batch.h:297-418) */
int bz_cm_batch_filter(bz_cache_manager_t* cm, int batch_id, const uint32_t* keep, uint32_t n_keep);
/* append src's sequences to dst; src ceases to exist (batch.h:482-576) */
int bz_cm_batch_extend(bz_cache_manager_t* cm, int dst_batch_id, int src_batch_id);
int bz_cm_batch_release(bz_cache_manager_t* cm, int batch_id);
/* host pointers into the batch's blob; valid until the batch changes */
int bz_cm_batch_table(bz_cache_manager_t* cm, int batch_id, const int32_t** indices_h, uint32_t* nnz_pages,
                      const int32_t** indptr_h, const int32_t** last_page_len_h, uint32_t* batch);
int bz_cm_stats(bz_cache_manager_t* cm, uint64_t* free_pages, uint64_t* allocated_pages, uint64_t* total_pages);
int bz_cm_pool(bz_cache_manager_t* cm, void** base, uint64_t* bytes);

/* library / device identification: "gfx950" build string, and hipGetErrorString passthrough */
const char* bz_build_info(void);
const char* bz_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* BZ_HIP_H_ */
