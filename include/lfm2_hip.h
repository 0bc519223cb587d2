/* C ABI of the gfx950 kernels behind the LFM2 continuous-batching decode/prefill step.
 *
 * The reference (lms21a/climbing-gym) has no FFI for this path: its seam is the set of
 * module-level Python functions that launch Triton kernels or call FlashAttention.  Each
 * entry point below replaces one of those functions; the comment names it as
 * file:line under src/climbing_gym/inference/ of the reference.
 *
 * Conventions
 *   - every pointer is a device pointer unless stated; tensors are row-major contiguous
 *     unless strides are passed;
 *   - `stream` is a hipStream_t; launches are stream-ordered, never synchronise, never
 *     allocate, and can be recorded into a hipGraph;
 *   - `dtype` is one of LFM2_DTYPE_*; fp8 means OCP e4m3 (finite only, max 448);
 *   - return value: LFM2_OK, or a negative code with text in lfm2_last_error().
 */
#ifndef LFM2_HIP_H
#define LFM2_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { LFM2_OK = 0, LFM2_ERR_ARGUMENT = -1, LFM2_ERR_LAUNCH = -2, LFM2_ERR_UNSUPPORTED = -3 };
enum { LFM2_DTYPE_BF16 = 0, LFM2_DTYPE_F16 = 1, LFM2_DTYPE_F32 = 2 };

const char* lfm2_last_error(void);
int lfm2_abi_version(void);

/* ---------------------------------------------------------------- embedding / norms / MLP glue */

/* F.embedding(tokens, table) of lfm25_cuda.py:134.  tokens int64[M], table [V,H] -> out [M,H]. */
int lfm2_embedding(void* out, const void* table, const int64_t* tokens, int64_t M, int64_t H, int64_t V,
                   int dtype, void* stream);

/* rms_norm of lfm25_cuda_kernels.py:32-55.  residual may be NULL (then summed is ignored).
 * out = round(x' * rsqrt(mean(x'^2)+eps)) * w with x' = round(x + residual); summed = x'. */
int lfm2_rms_norm(void* out, void* summed, const void* x, const void* weight, const void* residual,
                  int64_t M, int64_t H, float eps, int dtype, void* stream);

/* rms_norm_fp8 of lfm25_fp8.py:27-41,57-64: same, then per-row e4m3 with scale=max(amax/448,1e-12).
 * q uint8[M,H], scales float[M]. */
int lfm2_rms_norm_fp8(uint8_t* q, float* scales, void* summed, const void* x, const void* weight,
                      const void* residual, int64_t M, int64_t H, float eps, int dtype, void* stream);

/* rms_norm_fp8 whose input x[M,H] is given as split-K partial products of an FP8 projection:
 * x = round((sum_s partial[s]) * a_scales[m] * w_scales[h]) in the model dtype, i.e. what lfm2_fp8_gemm would have
 * stored; then exactly lfm2_rms_norm_fp8.  Fuses the projection's reduce pass into the norm that follows it in
 * lfm25_cuda.py:166-184.  (a_scales and w_scales both NULL: partial products of a bf16 projection, no scaling.) */
int lfm2_rms_norm_fp8_split(uint8_t* q, float* scales, void* summed, const float* partial, int splits,
                            const float* a_scales, const float* w_scales, const void* weight, const void* residual,
                            int64_t M, int64_t H, float eps, int dtype, void* stream);

/* rms_norm (model-dtype output) over the same kind of input; a_scales and w_scales both NULL for the partial
 * products of a bf16 projection (lfm2_bf16_gemm_partials), whose value is round(sum_s partial[s]).  The fused
 * add + norm of lfm25_cuda_kernels.py:32-55 with the projection's reduce pass folded in. */
int lfm2_rms_norm_split(void* out, void* summed, const float* partial, int splits, const float* a_scales,
                        const float* w_scales, const void* weight, const void* residual, int64_t M, int64_t H, float eps,
                        int dtype, void* stream);

/* F.embedding followed by the first layer's norm (lfm25_cuda.py:134-137: the first rms_norm of a step has no
 * residual) in one launch: hidden [M,H] receives the embedding rows (the residual stream), and either out [M,H]
 * (rms_norm) or q uint8[M,H] with scales float[M] (rms_norm_fp8) their norm.  Same bytes as the two launches. */
int lfm2_embedding_rms_norm(void* out, uint8_t* q, float* scales, void* hidden, const void* table, const int64_t* tokens,
                            const void* weight, int64_t M, int64_t H, int64_t V, float eps, int dtype, void* stream);

/* swiglu of lfm25_cuda_kernels.py:58-72.  x [M,2I] (gate first) -> out [M,I]. */
int lfm2_swiglu(void* out, const void* x, int64_t M, int64_t I, int dtype, void* stream);

/* swiglu_fp8 of lfm25_fp8.py:45-54,67-73. */
int lfm2_swiglu_fp8(uint8_t* q, float* scales, const void* x, int64_t M, int64_t I, int dtype, void* stream);

/* quantize_rows of lfm25_fp8.py:17-23,108-117.  x [M,K] -> q uint8[M,K], scales float[M]. */
int lfm2_quantize_rows(uint8_t* q, float* scales, const void* x, int64_t M, int64_t K, int dtype, void* stream);

/* conv_update of lfm25_cuda_kernels.py:75-110.  bcx [M,3H] in (B,C,x) thirds, weight [H,3],
 * state [slots,H,3] updated in place for active rows; active uint8[M] or NULL; slot_ids int32[M]
 * or NULL (negative ids read slot 0 and must be inactive). */
int lfm2_conv_update(void* out, const void* bcx, const void* weight, void* state, const uint8_t* active,
                     const int32_t* slot_ids, int64_t M, int64_t H, int64_t slots, int dtype, void* stream);

/* conv_update followed by quantize_rows of its output (lfm25_cuda.py:146-149 with an FP8 out projection) in one
 * launch: q uint8[M,H], scales float[M]; the values quantised are the model-dtype roundings lfm2_conv_update
 * stores.  H <= 4096. */
int lfm2_conv_update_fp8(uint8_t* q, float* scales, const void* bcx, const void* weight, void* state,
                         const uint8_t* active, const int32_t* slot_ids, int64_t M, int64_t H, int64_t slots,
                         int dtype, void* stream);

/* prepare_qkv of lfm25_cuda_kernels.py:113-151.  x [M,(QH+2KH)*D]; cos/sin float[P,D/2];
 * positions int32[M] -> q [M,QH,D], k [M,KH,D], v [M,KH,D]. */
int lfm2_prepare_qkv(void* q, void* k, void* v, const void* x, const void* q_weight, const void* k_weight,
                     const float* cos, const float* sin, const int32_t* positions, int64_t M, int QH, int KH,
                     int D, int64_t max_positions, float eps, int dtype, void* stream);

/* prepare_qkv followed by the decode-step KV append (store_kv of lfm25_fp8_kv.py:58-94 when kv_fp8, append_bf16_kv of
 * lfm25_adaptive.py:66 otherwise) in one launch: q [M,QH,D] is returned, the rotated keys and the values of row m go
 * to cache position positions[m] of slot slot_ids[m] (or m) unless the row is inactive, its slot id negative or its
 * position negative.  Caches are addressed as slot*c0 + position*c1 + head*c2 (elements); e4m3 scales sit at that
 * address divided by D.  D in {32,64,128,256}. */
int lfm2_prepare_qkv_store(void* q, const void* x, const void* q_weight, const void* k_weight, const float* cos,
                           const float* sin, const int32_t* positions, void* k_cache, void* v_cache, float* k_scales,
                           float* v_scales, const uint8_t* active, const int32_t* slot_ids, int64_t M, int QH, int KH,
                           int D, int64_t max_positions, float eps, int64_t c0, int64_t c1, int64_t c2, int kv_fp8,
                           int dtype, void* stream);

/* Packed-prefill short conv (F.conv1d path of lfm25_engine.py:1478-1511 on a varlen batch).
 * bcx [T,3H]; seq_of_token/pos_of_token int32[T]; seq_start int32[nseq+1] (cu_seqlens);
 * out [T,H]; state rows state[slots[seq]] receive the last three b*x of each sequence
 * (zero filled for shorter ones). */
int lfm2_conv_prefill(void* out, void* state, const void* bcx, const void* weight, const int32_t* cu_seqlens,
                      const int32_t* seq_of_token, const int32_t* slots, int64_t T, int64_t nseq, int64_t H,
                      int64_t nslots, int dtype, void* stream);

/* lfm2_conv_prefill followed by lfm2_quantize_rows (lfm25_fp8.py:108-117) in one launch, the same bits: the rows leave
 * as e4m3 codes q [T,H] with one fp32 scale per token, for an out projection that takes quantised activations
 * (PackedFP8Weight.linear_quantized, lfm25_fp8.py:141-168).  H % 8 == 0, H <= 2048, 16-bit dtype. */
int lfm2_conv_prefill_fp8(uint8_t* q, float* scales, void* state, const void* bcx, const void* weight,
                          const int32_t* cu_seqlens, const int32_t* seq_of_token, const int32_t* slots, int64_t T,
                          int64_t nseq, int64_t H, int64_t nslots, int dtype, void* stream);

/* ---------------------------------------------------------------- GEMMs */

/* PackedFP8Weight.linear_quantized of lfm25_fp8.py:77-105,141-168:
 * out[M,N] = (a_q[M,K] . w_q[N,K]^T) * a_scales[m] * w_scales[n], e4m3 x e4m3 -> fp32 MFMA.
 * workspace: float[split_k*M*N] when split_k > 1 (NULL otherwise); split_k <= 0 picks a default.
 * tile < 0 picks a default tile shape, otherwise an index into the table in gemm.hip. */
int lfm2_fp8_gemm(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                  const float* w_scales, float* workspace, int64_t M, int64_t N, int64_t K, int out_dtype,
                  int tile, int split_k, void* stream);
/* The QKV projection of an attention layer at decode with lfm2_prepare_qkv_store as its epilogue (head_dim 64, bf16,
 * K a multiple of 128): x_q[M,K] . w_q[(QH+2KH)*64, K]^T scaled and rounded to bf16 as lfm2_fp8_gemm stores it, then
 * per head QK-norm + RoPE, q [M,QH,64] written, keys and values appended to the cache at positions[m] (e4m3 with one
 * scale per token and head when kv_fp8, else the model dtype).  Bit for bit the two launches it replaces
 * (lfm25_fp8.py:141-168 then lfm25_cuda_kernels.py:113-151 and lfm25_fp8_kv.py:58-69 / lfm25_batching.py:49-69). */
int lfm2_fp8_gemm_qkv_store(void* q, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q, const float* w_scales,
                            const void* q_weight, const void* k_weight, const float* cos, const float* sin,
                            const int32_t* positions, void* k_cache, void* v_cache, float* k_scales, float* v_scales,
                            const uint8_t* active, const int32_t* slot_ids, int64_t M, int QH, int KH, int D, int64_t K,
                            int64_t max_positions, float eps, int64_t c0, int64_t c1, int64_t c2, int kv_fp8, int dtype,
                            void* stream);
/* The same product left as split-K partial sums: partials float[split_k, M, N], unscaled (no activation or weight
 * scale applied), split s covering its contiguous share of K.  For a consumer that folds the reduction into its own
 * pass (lfm2_rms_norm_fp8_split).  No counterpart in the reference, which always materialises the projection. */
int lfm2_fp8_gemm_partials(float* partials, const uint8_t* a_q, const uint8_t* w_q, int64_t M, int64_t N, int64_t K,
                           int tile, int split_k, void* stream);
/* Split count to give lfm2_fp8_gemm_partials for a shape (the tile it then picks suits that count); 1 = leave the
 * product whole with lfm2_fp8_gemm. */
int64_t lfm2_fp8_gemm_default_splits(int64_t M, int64_t N, int64_t K);
/* Workspace floats lfm2_fp8_gemm needs for a shape under its default choice (0 = none). */
int64_t lfm2_fp8_gemm_workspace(int64_t M, int64_t N, int64_t K);

/* linear of lfm25_cuda_kernels.py:19-29 (F.linear / GEMV): out[M,N] = x[M,K] . w[N,K]^T, bf16 in,
 * fp32 MFMA accumulate, bf16 out. */
int lfm2_bf16_gemm(void* out, const void* x, const void* w, float* workspace, int64_t M, int64_t N, int64_t K,
                   int tile, int split_k, void* stream);
int64_t lfm2_bf16_gemm_workspace(int64_t M, int64_t N, int64_t K);
/* The bf16 product left as split-K partial sums, float[split_k, M, N] (see lfm2_fp8_gemm_partials), and the split
 * count to give lfm2_bf16_gemm_partials for a shape (1 = leave the product whole).  No counterpart in the reference. */
int lfm2_bf16_gemm_partials(float* partials, const void* x, const void* w, int64_t M, int64_t N, int64_t K, int tile,
                            int split_k, void* stream);
int64_t lfm2_bf16_gemm_default_splits(int64_t M, int64_t N, int64_t K);

/* The gate+up projection with SwiGLU as its epilogue: w[N, K] is the packed weight [gate rows; up rows] (N = 2 I) in
 * the layout lfm2_fp8_gemm / lfm2_bf16_gemm read; out[M, I] = round(round(silu(gate)) * up) with gate and up the
 * product's columns rounded to the output type first, i.e. bit for bit lfm2_fp8_gemm (lfm25_fp8.py:141-168) or
 * lfm2_bf16_gemm followed by lfm2_swiglu (lfm25_cuda_kernels.py:58-72), without the [M, 2 I] intermediate.  Built on
 * one tile shape: lfm2_gemm_swiglu_fits(M, N, K, element bytes of the operands: 1 or 2) says whether a shape has the
 * fused form (1) or needs the two launches (0); the fused entry points return LFM2_ERR_UNSUPPORTED for the latter. */
int lfm2_gemm_swiglu_fits(int64_t M, int64_t N, int64_t K, int element_bytes);
int lfm2_fp8_gemm_swiglu(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q, const float* w_scales,
                         int64_t M, int64_t N, int64_t K, int out_dtype, void* stream);
int lfm2_bf16_gemm_swiglu(void* out, const void* x, const void* w, int64_t M, int64_t N, int64_t K, void* stream);

/* The conv in-projection with the gated short-conv update as its epilogue (decode): w[N, K] is the packed in-projection
 * weight [B rows; C rows; x rows] (N = 3 H); out[M, H] and the in-place update of state[slots, H, 3] are bit for bit
 * lfm2_fp8_gemm / lfm2_bf16_gemm followed by lfm2_conv_update (lfm25_cuda_kernels.py:75-110) with the same active and
 * slot_ids arguments, without the [M, 3 H] intermediate.  Built on one tile shape: lfm2_gemm_conv_fits(M, N, K, element
 * bytes of the operands) says whether a shape has the fused form; LFM2_ERR_UNSUPPORTED otherwise. */
int lfm2_gemm_conv_fits(int64_t M, int64_t N, int64_t K, int element_bytes);
int lfm2_fp8_gemm_conv_update(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q, const float* w_scales,
                              const void* conv_weight, void* state, const uint8_t* active, const int32_t* slot_ids,
                              int64_t M, int64_t N, int64_t K, int64_t slots, int out_dtype, void* stream);
int lfm2_bf16_gemm_conv_update(void* out, const void* x, const void* w, const void* conv_weight, void* state,
                               const uint8_t* active, const int32_t* slot_ids, int64_t M, int64_t N, int64_t K,
                               int64_t slots, void* stream);

/* The two products with placed output rows: row m of the product is written to out row out_rows[m] (m itself when
 * out_rows is NULL) unless that index is negative or >= out_capacity, or row_active[m] is 0 (row_active may be
 * NULL); other rows of out keep their contents.  This is the head projection followed by _scatter_logits of
 * lfm25_batching.py:25-32 (lfm25_cuda.py:190-192, lfm25_batching.py:99-101) in one launch, without the copy of
 * the logits.  Never split along K. */
int lfm2_fp8_gemm_rows(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q, const float* w_scales,
                       const int32_t* out_rows, const uint8_t* row_active, int64_t out_capacity, int64_t M, int64_t N,
                       int64_t K, int out_dtype, int tile, void* stream);
int lfm2_bf16_gemm_rows(void* out, const void* x, const void* w, const int32_t* out_rows, const uint8_t* row_active,
                        int64_t out_capacity, int64_t M, int64_t N, int64_t K, int tile, void* stream);

/* ---------------------------------------------------------------- KV cache and attention */

/* store_kv of lfm25_fp8_kv.py:28-69.  k,v [B,T,KH,D] with element strides (ks0,ks1,ks2) / (vs0,..);
 * caches e4m3 addressed slot*c0 + pos*c1 + head*c2 + d, scales float at the same offset / D.
 * positions int32[B] or NULL (then pos = token index), active uint8[B] or NULL, slot_ids or NULL. */
int lfm2_store_kv_fp8(const void* k, const void* v, uint8_t* k_cache, uint8_t* v_cache, float* k_scales,
                      float* v_scales, const int32_t* positions, const uint8_t* active, const int32_t* slot_ids,
                      int64_t B, int64_t T, int KH, int D, int64_t ks0, int64_t ks1, int64_t ks2, int64_t vs0,
                      int64_t vs1, int64_t vs2, int64_t c0, int64_t c1, int64_t c2, int dtype, void* stream);

/* append_bf16_kv of lfm25_batching.py:49-69 (also the in-kernel append of flash_attn_with_kvcache,
 * lfm25_cuda.py:161-165).  k,v [B,KH,D] contiguous; cache element strides (c0,c1,c2). */
int lfm2_append_kv(const void* k, const void* v, void* k_cache, void* v_cache, const int32_t* positions,
                   const int32_t* slot_ids, const uint8_t* active, int64_t B, int KH, int D, int64_t c0,
                   int64_t c1, int64_t c2, int dtype, void* stream);

/* Packed-prefill cache write (LFM25HybridCache.store_prefill, lfm25_engine.py:387-398) for a varlen
 * batch: token t goes to slot slots[seq_of_token[t]] at position t - cu_seqlens[seq].
 * kv_fp8 != 0 writes e4m3 + scales like lfm2_store_kv_fp8, otherwise copies in the model dtype. */
int lfm2_store_kv_packed(const void* k, const void* v, void* k_cache, void* v_cache, float* k_scales,
                         float* v_scales, const int32_t* cu_seqlens, const int32_t* seq_of_token,
                         const int32_t* slots, int64_t T, int KH, int D, int64_t c0, int64_t c1, int64_t c2,
                         int kv_fp8, int dtype, void* stream);

/* attend of lfm25_fp8_kv.py:72-167 (e4m3 history) and flash_attn_with_kvcache of
 * lfm25_cuda.py:156-165 (history in the model dtype, kv_fp8 = 0).
 * q [B,QH,D]; history rows [0, positions[b]] of slot slot_ids[b] (or b); out [B,QH,D];
 * inactive rows produce zeros.  block_table int32[B,max_blocks] or NULL: when given, token t of
 * row b lives in page block_table[b*max_blocks + t/page] at in-page index t%page and c0 is the
 * page stride (slot-mapped paged layout).  workspace: lfm2_decode_attention_workspace() floats (4-byte words). */
/* (out_q uint8[B,QH*D] with out_scales float[B], both or neither: when given, the rows are stored per-row e4m3
 * quantised, as lfm2_quantize_rows of the model-dtype result would, and `out` is not written.) */
int lfm2_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                          const float* k_scales, const float* v_scales, const int32_t* positions,
                          const uint8_t* active, const int32_t* slot_ids, const int32_t* block_table,
                          int64_t max_blocks, int page, const int32_t* schedule, float* workspace, int64_t B,
                          int QH, int KH, int D, int64_t capacity, int64_t c0, int64_t c1, int64_t c2, float scale,
                          int kv_fp8, int dtype, uint8_t* out_q, float* out_scales,
                          void* stream);
int64_t lfm2_decode_attention_workspace(int64_t B, int QH, int D, int64_t capacity);

/* Work list of the persistent decode-attention kernel: one (row, chunk) item per chunk of every active row's history
 * (chunks of 256 tokens, or of 512 when the batch would make at least 3072 chunks of 256), longest first (used for e4m3 and bf16 histories of head_dim 64 with GQA groups of at most 4 and
 * bf16 queries; other shapes ignore it).  It depends only on positions/active/slot_ids, so the attention layers of one
 * decode step can share it (pass it as `schedule`; NULL makes lfm2_decode_attention build its own in the workspace).
 * schedule: int32[lfm2_decode_schedule_size(B, capacity)].  No counterpart in the reference, whose Triton grid is
 * (rows, KV heads, splits) with a fixed split count (lfm25_fp8_kv.py:145-150). */
int lfm2_decode_schedule(int32_t* schedule, const int32_t* positions, const uint8_t* active, const int32_t* slot_ids,
                         int64_t B, void* stream);
int64_t lfm2_decode_schedule_size(int64_t B, int64_t capacity);
/* The head of a decode step in one launch (lfm25_cuda.py:128-133,185-186; with `slots`, lfm25_batching.py:11-22,35-46):
 * positions_out int32[B] = the rows' cache lengths before the step (row b's own slot, or slot slots[b]); the lengths
 * of the rows that take part advanced by one; the work list of lfm2_decode_schedule for those positions; and, with
 * `slots` (int32[B], -1 = padding), tokens_out int64[B] and mask_out uint8[B] gathered from input int64[slots] and
 * active uint8[slots] as lfm2_gather_inputs does.  Without `slots`, `active` is per row and may be NULL (all rows).
 * Equal to lfm2_gather_inputs + lfm2_decode_schedule before the layers and lfm2_advance_positions after them. */
int lfm2_decode_begin(int32_t* schedule, int32_t* positions_out, int64_t* tokens_out, uint8_t* mask_out, int32_t* lengths,
                      const int64_t* input, const uint8_t* active, const int32_t* slots, int64_t B, void* stream);

/* flash_attn_func(causal=True) of lfm25_engine.py:1415-1417 in varlen form: q [T,QH,D], k,v [T,KH,D]
 * packed by cu_seqlens int32[nseq+1]; out [T,QH,D]. */
int lfm2_prefill_attention(void* out, const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                           int64_t nseq, int64_t max_seqlen, int QH, int KH, int D, float scale, int dtype,
                           void* stream);

/* ---------------------------------------------------------------- batch metadata */

/* Expand cu_seqlens int32[nseq+1] into seq_of_token/pos_of_token int32[T] on the device
 * (replaces the host-side arange/indexing of lfm25_engine.py:659-662). */
int lfm2_build_token_map(int32_t* seq_of_token, int32_t* pos_of_token, const int32_t* cu_seqlens, int64_t nseq,
                         int64_t T, void* stream);

/* _gather_inputs of lfm25_batching.py:11-22. */
int lfm2_gather_inputs(int64_t* tokens, int32_t* positions, uint8_t* mask, const int64_t* input,
                       const int32_t* lengths, const uint8_t* active, const int32_t* slots, int64_t B,
                       void* stream);
/* _scatter_logits of lfm25_batching.py:25-32: saved[slots[row]] = logits[row] for active rows.
 * slots may be NULL (identity), which gives where(active, logits, saved) of lfm25_cuda.py:243. */
int lfm2_scatter_logits(void* saved, const void* logits, const int32_t* slots, const uint8_t* active, int64_t B,
                        int64_t V, int dtype, void* stream);
/* _advance_positions of lfm25_batching.py:35-46; slots NULL = identity (seq_lens.add_(active),
 * lfm25_cuda.py:185-186). */
int lfm2_advance_positions(int32_t* lengths, const int32_t* positions, const int32_t* slots,
                           const uint8_t* active, int64_t B, void* stream);

/* ---------------------------------------------------------------- sampling and bookkeeping */

/* sample_logits / RowSampler.sample of lfm25_sampling.py:9-123: greedy (temperature 0: first
 * maximum) or a draw from softmax(logits / T) over the full support (inverse CDF, one uniform per row;
 * the same law as the reference's Gumbel-max, V <= 2^20); logprobs are raw log-softmax of the pick,
 * sampling_logprobs (may be NULL) its log-probability under softmax(logits / T), the distribution drawn from
 * (greedy rows: the raw one; lfm25_engine.py:1591-1608).
 * Per-row arrays (seeds int64, steps int64, temperatures float) may be NULL, then the scalar
 * seed/step/temperature apply.  scratch: float[B*parts*4] with parts = ceil(V/4096). */
int lfm2_sample(int64_t* tokens, float* logprobs, float* sampling_logprobs, const void* logits, float* scratch,
                const int64_t* seeds, const int64_t* steps, const float* temperatures, int64_t seed, int64_t step,
                float temperature, int64_t B, int64_t V, int dtype, void* stream);

/* lfm2_sample without the scratch argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the tile statistics go to a file-scope device array
 * of 256 KiB that each GPU holds until the process ends.  No counterpart in the reference.  It allocates nothing and
 * calls nothing that allocates; B * ceil(V / 4096) must not exceed 16384 (e.g. 1024 rows of 65536 logits), larger
 * calls are refused with LFM2_ERR_ARGUMENT.  Every call on a GPU shares that GPU's array: calls that overlap on one
 * GPU (two streams) race; calls ordered on one stream do not, and nothing of an earlier call's contents is read.
 * The first call on a device looks the array's address up (hipGetSymbolAddress) and must come outside a capture. */
int lfm2_sample_static(int64_t* tokens, float* logprobs, const void* logits, const int64_t* seeds, const int64_t* steps,
                       const float* temperatures, int64_t seed, int64_t step, float temperature, int64_t B, int64_t V,
                       int dtype, void* stream);

/* _sample + _apply_top_k_top_p of lfm25_engine.py:1574-1609,1759-1774 on the device: temperature,
 * top-k (ties with the k-th value kept), nucleus (rank 0 never dropped), then a Gumbel-max draw
 * from what is left.  kept_count int32[B] (may be NULL) reports the survivors; sampling_logprobs float[B] (may be
 * NULL) the pick's log-probability under the tempered, filtered distribution (lfm25_engine.py:1605-1608).
 * temperatures float[B], top_ks int32[B], top_ps float[B] (all three or none) give every row its own parameters and
 * replace the scalars; a row whose parameters ask for no filter (top_k 0 and top_p 1) or for greedy decoding
 * (temperature 0) is then skipped and its outputs keep their contents (the sampler for those rows is lfm2_sample). */
int lfm2_sample_filtered(int64_t* tokens, float* logprobs, float* sampling_logprobs, int32_t* kept_count, const void* logits,
                         const int64_t* seeds, const int64_t* steps, const float* temperatures, const int32_t* top_ks,
                         const float* top_ps, int64_t seed, int64_t step, float temperature, int top_k, float top_p,
                         int64_t B, int64_t V, int dtype, void* stream);

/* _head_logprobs of lfm25_sampling.py:126-149: out[b,j] = values[b,j] - logZ(b). */
int lfm2_head_logprobs(float* out, const void* logits, const int64_t* selected, const float* logprobs,
                       const void* values, int64_t B, int64_t V, int K, int dtype, void* stream);

/* _record_sample of lfm25_session.py:34-56. */
int lfm2_record_sample(const int64_t* sampled, const float* logp, int64_t* tokens, float* logprobs,
                       int32_t* lengths, const int32_t* limits, int8_t* reasons, uint8_t* alive,
                       uint8_t* pending, int64_t* input, int64_t* stop_states, const int64_t* stop_offsets,
                       const int32_t* stop_table, const uint8_t* ignore_eos, int64_t* rng_positions,
                       int64_t eos, int64_t V, int64_t cap, int64_t B, void* stream);
/* lfm2_sample with per-row seeds, steps and temperatures, followed by lfm2_record_sample of its draw, in the sampler's
 * own launches (lfm25_session.py:469-482: RowSampler.sample, then _record_sample): sampled int64[B] and logp float[B]
 * receive the draw as from lfm2_sample; the record arguments are those of lfm2_record_sample.  `steps` may be the
 * same array as `rng_positions`: a row's step is read before its position is advanced. */
int lfm2_sample_record(int64_t* sampled, float* logp, const void* logits, float* scratch, const int64_t* seeds,
                       const int64_t* steps, const float* temperatures, int64_t* tokens, float* logprobs, int32_t* lengths,
                       const int32_t* limits, int8_t* reasons, uint8_t* alive, uint8_t* pending, int64_t* input,
                       int64_t* stop_states, const int64_t* stop_offsets, const int32_t* stop_table,
                       const uint8_t* ignore_eos, int64_t* rng_positions, int64_t eos, int64_t cap, int64_t B, int64_t V,
                       int dtype, void* stream);
/* The per-row state of newly admitted session requests (the state tensors of lfm25_session.py:150-165 as they are set
 * per request at :244-262) written in one launch: specs int64[count, 8] = slot, length limit, seed, random-stream
 * position, stop-automaton state, stop-table offset, flags (bit 0 ignore EOS, bits 8..39 top_k), temperature | top_p
 * (float bit patterns, low | high word).  Row `slot` of every column is set; length and finish reason become 0, the
 * row alive and not pending.  Specs whose slot is outside [0, rows) are ignored. */
int lfm2_configure_rows(const int64_t* specs, int64_t count, int64_t rows, int32_t* lengths, int32_t* limits,
                        int8_t* reasons, uint8_t* alive, uint8_t* pending, uint8_t* ignore_eos, float* temperatures,
                        int32_t* top_ks, float* top_ps, int64_t* seeds, int64_t* rng_positions, int64_t* stop_states,
                        int64_t* stop_offsets, void* stream);
/* _record_head of lfm25_session.py:22-31. */
int lfm2_record_head(const int64_t* ids, const float* probs, int32_t* out_ids, float* out_probs,
                     const int32_t* lengths, const uint8_t* alive, int K, int64_t cap, int64_t B, void* stream);

/* ---------------------------------------------------------------- measurement */

/* Loads-only streaming read of `bytes` bytes at src (16-byte aligned) by `workgroups` workgroups of 256 lanes, eight
 * 16-byte loads in flight per lane: the read rate the chip delivers to CUs that do nothing else, which bench.py
 * reports as the measured ceiling next to the nominal HBM peak.  No counterpart in the reference (its harness,
 * inference/benchmark.py:111-139, reports wall-clock phases only).  layout 0: every workgroup reads a private
 * contiguous region of floor(bytes / 4096 / workgroups) blocks of 4 KiB; layout 1: the grid sweeps the buffer together.
 * sink: int32[workgroups * 256], receives one folded word per lane.  Bytes read = workgroups * that many blocks * 4096. */
int lfm2_hbm_stream_read(const void* src, int64_t bytes, int32_t* sink, int workgroups, int layout, void* stream);

/* Register-operand loop of v_mfma_f32_16x16x128_f8f6f4 (e4m3): every wave of `workgroups` x `waves` (4, 8 or 16) issues
 * `iterations` rounds of eight independent instructions, 8 x 65536 flop each per round.  The dense fp8 rate the matrix
 * units deliver with nothing else in the way, which bench.py reports as the measured peak next to the nominal
 * 5.0 PFLOP/s when it gives the prefill products' MFMA utilisation.  No counterpart in the reference.
 * sink: float[workgroups * waves * 64]; clock: int64[2 * workgroups] or NULL, receives per workgroup the core clock
 * cycles and the constant-rate (lfm2_timestamp_rate_khz) ticks its first wave spent in the loop. */
int lfm2_mfma_fp8_peak(float* sink, int64_t* clock, int workgroups, int waves, int iterations, void* stream);

/* Stores the device's constant-rate wall clock into out[0] from a one-lane kernel; lfm2_timestamp_rate_khz() is the
 * clock's rate (0 if it cannot be read).  Recorded into a graph before and after a kernel, two stamps give that
 * kernel's time inside the replayed graph, which is how bench.py reads the decode-attention call's time inside the
 * decode step (the reference reads per-phase CUDA events, lfm25_session.py:184-204; event-record nodes are not
 * available to graphs captured through PyTorch on ROCm). */
int lfm2_timestamp(int64_t* out, void* stream);
int64_t lfm2_timestamp_rate_khz(void);

#ifdef __cplusplus
}
#endif
#endif
