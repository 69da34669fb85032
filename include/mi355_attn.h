/*
 * mi355_attn.h -- C ABI of libmi355attn.so: the attention hot path (causal
 * prefill forward + paged-KV decode) as hand-written HIP kernels for gfx950.
 *
 * Conventions shared by every entry point
 *   - all data pointers are DEVICE pointers owned by the caller; the library
 *     never allocates or frees device memory and never synchronises the host;
 *   - all work is enqueued on `stream` (a hipStream_t passed as void*; NULL is
 *     the default stream);
 *   - the return value is 0 on success, a negative MI355_E* code for a rejected
 *     argument, or a positive hipError_t from the launch; mi355_last_error()
 *     returns a thread-local message for the last non-zero return;
 *   - strides are in ELEMENTS; the innermost (head_dim) stride is always 1;
 *   - head_dim in {32, 64, 128}; GQA: query head h reads kv head h / (Hq / Hkv).
 */
#ifndef MI355_ATTN_H
#define MI355_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    MI355_OK = 0,
    MI355_EINVAL = -1,      /* bad shape / unsupported head_dim / null pointer   */
    MI355_EWORKSPACE = -2,  /* workspace too small                               */
    MI355_EDTYPE = -3       /* unsupported dtype code                            */
};

/* element type codes */
enum {
    MI355_BF16 = 0,         /* bfloat16 q/k/v/out and bf16 KV cache              */
    MI355_FP8_E4M3 = 1,     /* OCP fp8-e4m3 KV cache (max 448) + fp32 scales     */
    MI355_FP32 = 2          /* float32 (RMSNorm weight only)                     */
};

/* mask modes of the prefill entry point */
enum {
    MI355_MASK_NONE = 0,
    MI355_MASK_CAUSAL = 1,  /* query i keeps key j iff j <= i + (Sk - Sq)        */
    MI355_MASK_BOOL = 2     /* explicit uint8 keep-mask (non-zero = attend)      */
};

/*
 * Prefill attention forward: out = softmax(q k^T * softmax_scale [masked]) v.
 *
 * Replaces, in the reference, the attention slot of
 * CausalMultiHeadSelfAttention.forward -- llm-core/llm_core/model.py:380-385 --
 * i.e. torch.nn.functional.scaled_dot_product_attention(Q, K, V, is_causal=True)
 * (model.py:382) and scaled_dot_product_attention(Q, K, V, mask)
 * (model.py:308-325, softmax at llm-core/llm_core/nn_functional.py:8-11).
 *
 * Dense layout (cu_seqlens_q == NULL): tensors are (B, H, S, D) addressed as
 *   base + b*strides[0] + h*strides[1] + s*strides[2] + d, so the reference's
 *   contiguous Q/K and its strided V view (model.py:367-370) are both accepted.
 * Packed layout (cu_seqlens_q != NULL): tensors are (T, H, D) addressed as
 *   base + t*strides[2] + h*strides[1] + d (strides[0] ignored); sequence b
 *   owns rows [cu_seqlens[b], cu_seqlens[b+1]); cu_seqlens are int32 (B+1).
 * mask (MI355_MASK_BOOL only): uint8, element (b,h,i,j) at
 *   mask + b*mask_strides[0] + h*mask_strides[1] + i*mask_strides[2] + j
 *   (use stride 0 to broadcast); dense layout only.  A query row with every key
 *   masked yields NaN, as the reference's softmax does.
 * Sq_max/Sk_max: the (maximum) query/key sequence lengths.
 */
int mi355_prefill_fwd(const void* q, const void* k, const void* v, void* out,
                      const int64_t q_strides[3], const int64_t k_strides[3],
                      const int64_t v_strides[3], const int64_t o_strides[3],
                      const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                      const uint8_t* mask, const int64_t mask_strides[3],
                      int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                      float softmax_scale, int mask_mode, int dtype, void* stream);

/*
 * Prefill forward that also returns the log-sum-exp of every query row, which the backward
 * needs: lse[b,h,i] = log sum_j exp(softmax_scale * q_i.k_j) over the kept keys (natural log,
 * fp32; -inf for a row with no kept key).  lse is addressed as
 *   dense : lse + b*lse_strides[0] + h*lse_strides[1] + i
 *   packed: lse + h*lse_strides[1] + t            (t = row in the packed query buffer)
 * Same computation and arguments as mi355_prefill_fwd otherwise (mask modes NONE / CAUSAL).
 * This is the forward half of what torch.nn.functional.scaled_dot_product_attention does under
 * autograd at llm-core/llm_core/model.py:382 when train.py runs with --flash-attn (train.py:312).
 */
int mi355_prefill_fwd_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                          const int64_t q_strides[3], const int64_t k_strides[3],
                          const int64_t v_strides[3], const int64_t o_strides[3],
                          const int64_t lse_strides[2],
                          const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                          int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                          float softmax_scale, int mask_mode, int dtype, void* stream);

/*
 * Causal prefill of a CHUNK of new tokens on top of context that is already in a paged bf16 cache
 * (chunked prefill / prefix reuse; an fp8 cache: mi355_gather_kv_fp8 below).  The keys and values of all context_lens[b] tokens of sequence b
 * -- the chunk's own included: write them first with mi355_rope_and_cache -- are read through
 * block_tables (the layout of mi355_paged_decode_fwd: int32 (B, table_stride), entry j = physical
 * block of tokens [16j, 16j+16); k_cache/v_cache (num_blocks,Hkv,16,D) bf16).  The chunk's queries
 * are packed: q/out (T,Hq,D) with contiguous heads, sequence b owning rows
 * [cu_seqlens_q[b], cu_seqlens_q[b+1]); its query i keeps key j iff
 * j <= i + (context_lens[b] - chunk length), the bottom-right aligned mask of MI355_MASK_CAUSAL.
 * Only table entries of blocks that hold a valid key are read, and never more than max_blocks per row
 * (the width of the table, <= table_stride): a context_lens[b] beyond 16 * max_blocks is cut to it,
 * as mi355_paged_decode_fwd cuts one beyond max_ctx.  Sq_max = longest chunk.
 * Same mathematics as mi355_prefill_fwd (model.py:308-325 / :382) -- the reference has no cache,
 * so it has no counterpart of the table walk; what it replaces is re-running the whole prefix at
 * model.py:218 when a prompt arrives in pieces.
 * n_split > 1 splits every sequence's keys over n_split workgroups (see mi355_prefill_fwd_splitkv:
 * a short chunk over a long context would otherwise occupy a handful of compute units); it then needs
 * total_q_rows = cu_seqlens_q[B] and a workspace of mi355_prefill_splitkv_workspace_bytes().
 * n_split <= 1: workspace may be NULL.
 */
int mi355_prefill_paged_fwd(const void* q, const void* k_cache, const void* v_cache, void* out,
                            int64_t q_token_stride, int64_t out_token_stride,
                            const int32_t* cu_seqlens_q, const int32_t* block_tables, int64_t table_stride,
                            int64_t max_blocks, const int32_t* context_lens, int B, int Hq, int Hkv, int Sq_max,
                            int D, int block_size, int64_t num_blocks, float softmax_scale, int kv_dtype,
                            int n_split, int64_t total_q_rows, void* workspace, size_t workspace_bytes,
                            void* stream);

/*
 * The same chunk over an fp8-e4m3 cache goes in two steps: mi355_gather_kv_fp8 reads every sequence's keys
 * and values through the block tables and writes them dequantised -- bf16(fp8 * scale of the (block, kv
 * head) slab) -- as packed rows, k_out / v_out (rows, Hkv, D) bf16 with token stride out_token_stride,
 * sequence b owning rows [cu_seqlens_k[b], cu_seqlens_k[b+1]) (cu_seqlens_k = running sum of the context
 * lengths, int32 (B+1), on the device); mi355_prefill_fwd (or _splitkv) then runs on q with cu_seqlens_q
 * and on those rows with cu_seqlens_k -- the packed layout with more keys than queries per sequence,
 * bottom-right aligned causal mask -- on the same kernels as any bf16 prefill.
 * k_scale / v_scale: fp32 (num_blocks, Hkv) as in mi355_paged_decode_fwd.  max_blocks: width of the table
 * (a longer context_lens[b] is cut to 16 * max_blocks); rows at or past max_rows (the capacity of k_out /
 * v_out in rows) are not written.  block_size must be 16; D in {32, 64, 128}.
 * No reference counterpart (the reference has no cache).
 */
int mi355_gather_kv_fp8(const void* k_cache_fp8, const void* v_cache_fp8, const float* k_scale,
                        const float* v_scale, const int32_t* block_tables, int64_t table_stride,
                        int64_t max_blocks, const int32_t* context_lens, const int32_t* cu_seqlens_k,
                        void* k_out, void* v_out, int64_t out_token_stride, int64_t max_rows, int B, int Hkv,
                        int D, int block_size, int64_t num_blocks, void* stream);

/*
 * mi355_prefill_fwd with the keys of every sequence split over n_split workgroups (flash-decoding for
 * prefill): share c of a query tile's K/V tiles yields a normalised fp32 partial result and its
 * log-sum-exp per query row, and a second kernel merges them,
 *   out = sum_c w_c O_c / sum_c w_c,   w_c = exp(lse_c - max lse).
 * For few or short query sequences over long key sequences (one long prompt, a short chunk over a
 * long context), where one workgroup per pair of query tiles leaves most compute units idle.  The
 * partials cost 4 (D + 1) n_split bytes of traffic per query row and head each way, so splitting pays
 * when queries are few.  Same arguments as mi355_prefill_fwd (mask modes NONE / CAUSAL), plus:
 *   n_split       1..64 (1: plain mi355_prefill_fwd, no workspace needed)
 *   total_q_rows  B * Sq_max (dense) or the packed number of query rows
 *   workspace     >= mi355_prefill_splitkv_workspace_bytes(total_q_rows, Hq, D, n_split), 16-byte aligned
 * No reference counterpart beyond the mathematics of model.py:308-325.
 */
size_t mi355_prefill_splitkv_workspace_bytes(int64_t total_q_rows, int Hq, int D, int n_split);
/*
 * A good n_split for a forward prefill of this shape (1 = do not split): a host-side cost model fitted to
 * timings on an MI355X -- a share of the keys must save more tile-loop time than its fp32 partial rows cost in
 * traffic, so few query rows over many keys split 4..16 ways and a launch that fills the GPU is left alone.
 * Sq_max / Sk_max: longest query / key sequence; causal: non-zero for MI355_MASK_CAUSAL;
 * n_compute_units <= 0: ask the current device (the only case that touches the GPU runtime).
 */
int mi355_prefill_suggest_kv_splits(int B, int Hq, int D, int Sq_max, int Sk_max, int64_t total_q_rows,
                                    int causal, int n_compute_units);
int mi355_prefill_fwd_splitkv(const void* q, const void* k, const void* v, void* out,
                              const int64_t q_strides[3], const int64_t k_strides[3],
                              const int64_t v_strides[3], const int64_t o_strides[3],
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                              int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                              float softmax_scale, int mask_mode, int dtype,
                              int n_split, int64_t total_q_rows, void* workspace, size_t workspace_bytes,
                              void* stream);

/*
 * Prefill backward: dq, dk, dv of out = softmax(q k^T * softmax_scale [causal]) v given dout,
 * i.e. the gradient that autograd derives for the attention call at model.py:380-385
 * (model.py:308-325 is its definition) during loss.backward() (train.py:224).
 *   q, k, v, out, dout, dq, dk, dv : bf16, layouts and stride conventions of mi355_prefill_fwd
 *                                    (dq like q, dk/dv like k/v, dout like out), each with its own strides
 *   lse   : as written by mi355_prefill_fwd_lse for the same inputs
 *   delta : fp32 scratch with lse's layout and size (receives rowsum(dout * out))
 * GQA: dk/dv of a kv head sum over its Hq/Hkv query heads.  Mask modes NONE / CAUSAL.
 * A causal query row that sees no key (Sq > Sk) gets dq = 0.  Two launches on `stream`
 * (dq, which also fills delta; then dk and dv together); no atomics, so the result is deterministic.
 */
int mi355_prefill_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout,
                      const float* lse, float* delta, void* dq, void* dk, void* dv,
                      const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                      const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                      const int64_t dk_strides[3], const int64_t dv_strides[3], const int64_t lse_strides[2],
                      const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                      int B, int Hq, int Hkv, int Sq_max, int Sk_max, int D,
                      float softmax_scale, int mask_mode, int dtype, void* stream);

/*
 * The training pair for an explicit mask: what autograd needs behind
 * scaled_dot_product_attention(Q, K, V, mask) of model.py:308-325 as the reference's non-flash
 * branch calls it (model.py:384-385, under loss.backward() at train.py:224).
 * mi355_prefill_fwd_mask_lse is mi355_prefill_fwd in mode MI355_MASK_BOOL (dense layout only) that
 * also writes lse (layout as in mi355_prefill_fwd_lse; a row whose keys are all masked gets -inf
 * and a NaN output row, as the reference's softmax gives it).  mi355_prefill_bwd_mask is
 * mi355_prefill_bwd under the same mask: every tile takes the per-element select and fetches its
 * mask bytes, so it is the general path, slower than the causal one.  For the backward the mask
 * pointer and its three byte strides must be multiples of 4 (keys are fetched four at a time), and a
 * row must be readable up to the next multiple of 4 past Sk.  A fully masked row contributes zero
 * gradients (the reference propagates its NaN instead).
 */
int mi355_prefill_fwd_mask_lse(const void* q, const void* k, const void* v, void* out, float* lse,
                               const int64_t q_strides[3], const int64_t k_strides[3],
                               const int64_t v_strides[3], const int64_t o_strides[3],
                               const int64_t lse_strides[2], const uint8_t* mask,
                               const int64_t mask_strides[3], int B, int Hq, int Hkv, int Sq, int Sk, int D,
                               float softmax_scale, int dtype, void* stream);
int mi355_prefill_bwd_mask(const void* q, const void* k, const void* v, const void* out, const void* dout,
                           const float* lse, float* delta, void* dq, void* dk, void* dv,
                           const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                           const int64_t o_strides[3], const int64_t do_strides[3], const int64_t dq_strides[3],
                           const int64_t dk_strides[3], const int64_t dv_strides[3],
                           const int64_t lse_strides[2], const uint8_t* mask, const int64_t mask_strides[3],
                           int B, int Hq, int Hkv, int Sq, int Sk, int D, float softmax_scale, int dtype,
                           void* stream);

/*
 * Paged-KV decode attention, one query token per sequence (split-K + combine).
 *
 * No counterpart exists in the reference: it is what a KV-cached replacement of
 * TransformerLM.generate (llm-core/llm_core/model.py:187-236, which re-runs the
 * full forward per token at :218) calls every step.  Its result is defined by
 * reduction to model.py:308-325 on the gathered KV.
 *
 *   q, out        : (B, Hq, D) bf16, contiguous; Hq a multiple of Hkv (a kv head with more than 16
 *                   query heads is streamed once per 16 of them)
 *   k_cache/v_cache: (num_blocks, Hkv, block_size, D), bf16 (kv_dtype MI355_BF16)
 *                   or fp8-e4m3 bytes (MI355_FP8_E4M3); block_size must be 16
 *   block_tables  : int32, row b at block_tables + b*bt_row_stride; entry j is
 *                   the physical block of tokens [16j, 16j+16); entries past
 *                   ceil(context_lens[b]/16) are never read
 *   context_lens  : int32 (B), each >= 1 (0 leaves that row of `out` unwritten)
 *   k_scale/v_scale: fp32 (num_blocks, Hkv), required iff kv_dtype is fp8;
 *                   real value = fp8 value * scale
 *   workspace     : >= mi355_paged_decode_workspace_bytes(...) bytes, 16-byte
 *                   aligned, contents irrelevant on entry (split-K partials)
 *   num_blocks    : blocks in the pool; a table entry outside [0, num_blocks) is clamped into
 *                   the pool (the result for that sequence is then meaningless, but no
 *                   memory outside the caches is touched)
 *   max_ctx       : upper bound on every context_lens[b] (sizes the grid); a larger
 *                   context_lens[b] is truncated to it
 */
int mi355_paged_decode_fwd(const void* q, const void* k_cache, const void* v_cache, void* out,
                           const int32_t* block_tables, int64_t bt_row_stride,
                           const int32_t* context_lens,
                           const float* k_scale, const float* v_scale,
                           void* workspace, size_t workspace_bytes,
                           int B, int Hq, int Hkv, int D, int block_size, int64_t num_blocks, int max_ctx,
                           float softmax_scale, int kv_dtype, void* stream);

/* Workspace requirement of mi355_paged_decode_fwd.  Monotonic in every argument: a workspace sized for a
 * caller's largest batch and longest context serves every call with smaller ones. */
size_t mi355_paged_decode_workspace_bytes(int B, int Hq, int D, int max_ctx);

/*
 * mi355_paged_decode_fwd without a workspace argument and without any allocation: the split-K partials go to a
 * device array that is part of the library's own code object (MI355_STATIC_SCRATCH_BYTES per GPU, held from the
 * first load until the process ends).  It has no counterpart in the reference; it exists for callers that cannot
 * allocate or size a workspace: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments, kernels and results (bit for bit) as mi355_paged_decode_fwd otherwise.
 *   - a call whose partials need more than the array (mi355_paged_decode_workspace_bytes of the layout actually
 *     used, i.e. B * Hq * ceil(max_ctx / mi355_paged_decode_chunk_tokens(B, Hq, Hkv, max_ctx)) * (D + 2) * 4 bytes plus padding)
 *     is rejected with MI355_EWORKSPACE; max_ctx up to one chunk needs no scratch at all;
 *   - all calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 *     threads) race on it and must be serialised by the caller; the array's old contents never matter (every
 *     partial that the combine pass reads is written by the split pass of the same call);
 *   - the array's address is looked up on the first call on each device (not a stream operation); make that
 *     first call outside a graph capture, like the first launch of any kernel.
 */
#define MI355_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
int mi355_paged_decode_fwd_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                  const int32_t* block_tables, int64_t bt_row_stride,
                                  const int32_t* context_lens,
                                  const float* k_scale, const float* v_scale,
                                  int B, int Hq, int Hkv, int D, int block_size, int64_t num_blocks, int max_ctx,
                                  float softmax_scale, int kv_dtype, void* stream);

/* Tokens of one sequence handled by one workgroup of the split-K pass: grows with max_ctx (1024, 2048, 4096) and
 * shrinks again, down to 256, while a batch of contexts beyond 1024 tokens has fewer workgroups than the GPU has
 * compute units. */
int mi355_paged_decode_chunk_tokens(int B, int Hq, int Hkv, int max_ctx);

/*
 * RoPE + KV-cache write: the producer of the paged cache (the step right before the
 * attention path).  Rotates adjacent pairs (x[2i], x[2i+1]) of q and k by the angle of
 * (position, i) exactly as RotaryEmbedding.forward does -- llm-core/llm_core/model.py:93-104
 * -- reading cos/sin from the reference's own table layout `_freq_cache`
 * (2, context_length, D/2) fp32, model.py:86-91; fp32 math, one rounding to bf16.
 * The rotated queries go to q_out (may alias q_in); rotated keys and the unrotated values
 * of token t are scattered to cache slot slot_mapping[t] = block*16 + offset (negative:
 * token not cached; NULL slot_mapping: rotate q only... k/v are then ignored).
 * The scatter has no counterpart in the reference (it has no KV cache).
 *   q_in/q_out (T,Hq,D), k_in/v_in (T,Hkv,D) bf16, heads contiguous, token strides in elements;
 *   positions int32 (T), each < context_length (a position outside the table is clamped into it);
 *   k_cache/v_cache (num_blocks,Hkv,16,D) bf16; a slot outside [0, num_blocks*16) is not written;
 *   k_out (optional, else NULL): the rotated keys once more, packed (T,Hkv,D) bf16 with token stride
 *   k_out_token_stride -- the K operand of a prefill over the same tokens (mi355_prefill_fwd), so that
 *   one launch serves the cache and the prefill; may alias k_in.
 */
int mi355_rope_and_cache(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                         void* k_cache, void* v_cache, const float* freq_cache,
                         const int32_t* positions, const int64_t* slot_mapping, int64_t num_blocks,
                         int T, int Hq, int Hkv, int D, int context_length,
                         int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
                         int64_t q_out_token_stride, void* k_out, int64_t k_out_token_stride, void* stream);

/*
 * Per-(block, kv head) absmax quantisation of a bf16 cache (num_blocks,Hkv,16,D) to OCP
 * fp8-e4m3 bytes + fp32 scales (num_blocks,Hkv): scale = absmax/448 (1 for an all-zero
 * slab), value = round_to_nearest_even(clamp(x/scale, +-448)).  No reference counterpart;
 * it produces the cache format MI355_FP8_E4M3 of mi355_paged_decode_fwd.
 */
int mi355_quantize_kv_fp8(const void* cache_bf16, void* cache_fp8, float* scale,
                          int64_t num_blocks, int Hkv, int D, int block_size, void* stream);

/*
 * mi355_rope_and_cache with an fp8-e4m3 cache (the MI355_FP8_E4M3 format of
 * mi355_paged_decode_fwd): RoPE as in llm-core/llm_core/model.py:93-104, then the rotated keys
 * (rounded to bf16 first, as a bf16 cache would hold them) and the values are quantised into
 * k_cache_fp8 / v_cache_fp8 (num_blocks,Hkv,16,D) bytes, and k_scale / v_scale (num_blocks,Hkv)
 * fp32 are maintained so that a block's scale is always absmax/448 of its valid rows: writing
 * at offset 0 starts the block afresh; writing at a later offset keeps the scale or, when the new
 * rows raise it, re-expresses the rows already there in the new scale (fp8 -> fp32 -> fp8).
 * Tokens that share a block must be adjacent in the packed order with consecutive slots (a run),
 * and a block may receive one run per call (one sequence = one run per block, as a prefill or a
 * decode step produces them).  Slots outside [0, 16*num_blocks) are skipped.  Needs 16-byte
 * aligned tensors, token strides that are multiples of 8, D in {32, 64, 128}.  k_out (optional)
 * receives the rotated keys in bf16, packed (T,Hkv,D), as in mi355_rope_and_cache: a prefill over
 * the tokens of this call then attends to unquantised keys; unlike there it must NOT overlap k_in
 * (MI355_EINVAL): here the keys are read a second time, by other workgroups of the same launch, for
 * the quantised write.  No reference counterpart (the reference has no KV cache).
 */
int mi355_rope_and_cache_fp8(const void* q_in, const void* k_in, const void* v_in, void* q_out,
                             void* k_cache_fp8, void* v_cache_fp8, float* k_scale, float* v_scale,
                             const float* freq_cache, const int32_t* positions,
                             const int64_t* slot_mapping, int64_t num_blocks,
                             int T, int Hq, int Hkv, int D, int context_length,
                             int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
                             int64_t q_out_token_stride, void* k_out, int64_t k_out_token_stride,
                             void* stream);

/*
 * RMSNorm forward over the rows of a (n_rows, n_cols) bf16 matrix:
 *   y = weight * (h * rsqrt(mean(h^2) + eps)),  h = x, or h = bf16(x + residual)
 * fp32 math, one rounding to bf16 -- RMSNorm.forward, llm-core/llm_core/model.py:60-67, and the
 * forward of its Triton twin, llm-systems/llm_systems/kernels/triton_rms_norm.py:30-74.
 * `residual` (optional) fuses the residual add in front of the norm (TransformerBlock.forward,
 * model.py:293-294, adds and then normalises); `sum_out` (optional, needs residual) receives h;
 * `rstd_out` (optional, fp32 n_rows) receives 1/rms as the Triton kernel caches it (:68).
 * Row strides in elements; weight is bf16 (MI355_BF16) or fp32 (MI355_FP32), n_cols long.
 */
int mi355_rms_norm_fwd(const void* x, const void* residual, const void* weight, void* y, void* sum_out,
                       float* rstd_out, int64_t n_rows, int n_cols, int64_t x_row_stride,
                       int64_t residual_row_stride, int64_t y_row_stride, int64_t sum_row_stride, float eps,
                       int weight_dtype, void* stream);

/*
 * out = bf16(silu(gate)) * up over (n_rows, n_cols) bf16 matrices with row strides (elements):
 * silu in fp32, rounded to bf16, product rounded to bf16 -- _silu_mul_fwd_kernel,
 * llm-systems/llm_systems/kernels/triton_swiglu.py:27-47 (and SwiGLU.forward, model.py:304-305).
 * Strided rows let gate and up be the two halves of one merged projection output
 * (FusedSwiGLU.forward, triton_swiglu.py:190-194) without the copies made there.
 */
int mi355_silu_mul_fwd(const void* gate, const void* up, void* out, int64_t n_rows, int n_cols,
                       int64_t gate_row_stride, int64_t up_row_stride, int64_t out_row_stride, void* stream);

/*
 * Plain device-to-device copy of `bytes` bytes (16-byte aligned).  Measurement aid
 * with no counterpart in the reference: a copy of known size whose FETCH_SIZE /
 * WRITE_SIZE counter readings calibrate the HBM-traffic figures of the kernels above.
 */
int mi355_calib_copy(const void* src, void* dst, size_t bytes, void* stream);

const char* mi355_last_error(void);
const char* mi355_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_ATTN_H */
