/*
 * libmla_hip.so — C ABI of the gfx950 (MI355X) MLA / DSA attention kernels.
 *
 * Conventions for every entry point:
 *   - plain device pointers, sizes and strides; strides are in ELEMENTS of the tensor's dtype unless a
 *     parameter name ends in _bytes; the last dimension of every tensor is contiguous;
 *   - `stream` is a hipStream_t (PyTorch-ROCm: torch.cuda.current_stream().cuda_stream); work is only
 *     enqueued, nothing synchronises, nothing is allocated or freed, the library owns no memory;
 *   - returns 0 on success or a negative code (-1 null pointer, -2 bad size/stride/alignment,
 *     -3 unsupported, -4 workspace too small, -100 launch refused by the HIP runtime) and leaves a
 *     message for mlahip_last_error_string(); never throws;
 *   - int32 `seq_lens` / `block_table` / `query_start_loc` live on the device, so a captured HIP graph
 *     stays valid when their contents change between replays.
 * Paths cited below are relative to the reference tree (drago1234/omni-npu, src/omni_npu/...).
 */
#ifndef MLA_HIP_H
#define MLA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* mlahip_stream_t;

int mlahip_version(void);
const char* mlahip_last_error_string(void);

/* ---- latent-KV cache write ------------------------------------------------------------------
 * Replaces torch_npu.npu_scatter_nd_update_ in store_kv, attention/backends/mla.py:868-881 and
 * attention/backends/dsa.py:359-362:  cache.flatten(0,1)[slot[t]] = src[t]; slot = page * page_size + offset;
 * negative slots (padding) and slots past the cache are skipped. */
int mla_cache_write_bf16(const void* kv_c, int64_t kv_c_stride,           /* bf16 [T,512] */
                         const void* k_pe, int64_t k_pe_stride,           /* bf16 [T,64]  */
                         const int64_t* slot_mapping, int32_t num_tokens,
                         void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride, /* bf16 [pages,page,512] */
                         void* rope_cache, int64_t rope_page_stride, int64_t rope_row_stride, /* bf16 [pages,page,64]  */
                         int32_t page_size, int64_t num_pages, mlahip_stream_t stream);

/* One cache of any row width (a multiple of 16 bytes): the indexer-K scatter of
 * vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:116-121 and
 * v1/layers/attention/npu_dsa.py:134-139. */
int mla_scatter_rows(const void* src, int64_t src_stride_bytes, int32_t row_bytes, const int64_t* slot_mapping,
                     int32_t num_tokens, void* cache, int64_t page_stride_bytes, int64_t row_stride_bytes,
                     int32_t page_size, int64_t num_pages, mlahip_stream_t stream);

/* fp8-e4m3 block-scaled latent cache: one 656-byte row per token = 512 x e4m3 | 4 x fp32 scale
 * (scale = amax/448 per 128 elements, 1.0 for an all-zero block) | 64 x bf16 rope.  The reference has no fp8 KV
 * format (attention/ops.py:11-12 accepts and ignores a scale; mla.py:791-792 passes antiquant_mode=0), so the layout
 * is this library's own. */
int mla_cache_write_fp8(const void* kv_c, int64_t kv_c_stride, const void* k_pe, int64_t k_pe_stride,
                        const int64_t* slot_mapping, int32_t num_tokens, void* cache, int64_t page_stride_bytes,
                        int64_t row_stride_bytes, int32_t page_size, int64_t num_pages, mlahip_stream_t stream);

/* ---- the step in front of the path, fused ----------------------------------------------
 * Replaces torch_npu.npu_kv_rmsnorm_rope_cache as called at v1/layers/attention/npu_mla.py:196-206, 296-309 and
 * v1/layers/attention/npu_dsa.py:410-424, 517-527: RMSNorm(kv_a [T,512], gamma, eps) and the rotary embedding of
 * k_pe [T,64] written straight into the paged cache rows named by slot_mapping (negative / out-of-range slots are
 * skipped), plus, when the pointers are not NULL, the normalised latent and the rotated rope key as plain tensors
 * (is_output_kv=True); slot_mapping = NULL skips the cache altogether (both plain outputs are then required).
 * kv_a and k_pe are usually the two halves of one [T,576] tensor (k_pe = kv_a + 512).
 * Arithmetic (fp32, one rounding to bf16): y = x * rsqrt(mean(x^2) + eps) * gamma;
 * x1 = k_pe[0::2], x2 = k_pe[1::2], o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin with pair i reading table entry
 * i*cos_step of the token's cos / sin row (rows cs_stride elements apart): cos_step 1 for the reference's cat(c, c)
 * rows (layers/rotary_embedding/rotary_embedding_torch_npu.py:170-173), 2 for rows that repeat every entry.
 * interleaved_out = 0 stores cat(o1, o2) (the reference's result, rotary_embedding_torch_npu.py:146-163);
 * 1 stores the pairs back in place (GPT-J layout, tests/integration/attention/test_npu_mla_math.py:125-144). */
int mla_kv_rmsnorm_rope_cache(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                              const void* gamma /* bf16 [512] */, const void* cos, const void* sin, int64_t cs_stride,
                              int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping, int32_t num_tokens,
                              float eps, void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride,
                              void* rope_cache, int64_t rope_page_stride, int64_t rope_row_stride, int32_t page_size,
                              int64_t num_pages, void* kv_a_out /* may be NULL */, int64_t kv_a_out_stride,
                              void* k_pe_out /* may be NULL */, int64_t k_pe_out_stride, mlahip_stream_t stream);

/* Same, into the fp8-e4m3 block-scaled cache of mla_cache_write_fp8 (the bf16-rounded normalised row is quantised,
 * so the bytes equal mla_cache_write_fp8 applied to the outputs of the bf16 variant). */
int mla_kv_rmsnorm_rope_cache_fp8(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                  const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                  int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                  int32_t num_tokens, float eps, void* cache, int64_t page_stride_bytes,
                                  int64_t row_stride_bytes, int32_t page_size, int64_t num_pages, void* kv_a_out,
                                  int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride,
                                  mlahip_stream_t stream);

/* Replaces torch_npu.npu_interleave_rope (npu_mla.py:210, 316; npu_dsa.py:407, 528) for the query's rope part:
 * x [T, N, 64] through its strides -> out [T, N, 64], same rotation and table conventions as above.  In place
 * (out == x with the same strides) is allowed. */
int mla_interleave_rope(const void* x, int64_t x_stride_t, int64_t x_stride_h, int64_t num_tokens, int32_t num_heads,
                        const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step, int32_t interleaved_out,
                        void* out, int64_t out_stride_t, int64_t out_stride_h, mlahip_stream_t stream);

/* mla_kv_rmsnorm_rope_cache[_fp8] and mla_interleave_rope of the same tokens in ONE launch: the whole rotary / norm /
 * cache-write prologue of a decode step (npu_mla.py:196-210: the reference issues the two vendor ops back to back).
 * q [T, num_heads, 64] through its strides -> q_out (may be q itself, same strides); same tables and the same
 * interleaved_out convention for the key and the query. */
int mla_kv_rmsnorm_rope_cache_q(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                const void* gamma, const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step,
                                int32_t interleaved_out, const int64_t* slot_mapping, int32_t num_tokens, float eps,
                                void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride, void* rope_cache,
                                int64_t rope_page_stride, int64_t rope_row_stride, int32_t page_size, int64_t num_pages,
                                void* kv_a_out, int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride,
                                const void* q, int64_t q_stride_t, int64_t q_stride_h, int32_t num_heads, void* q_out,
                                int64_t q_out_stride_t, int64_t q_out_stride_h, mlahip_stream_t stream);
int mla_kv_rmsnorm_rope_cache_q_fp8(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                    const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                    int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                    int32_t num_tokens, float eps, void* cache, int64_t page_stride_bytes,
                                    int64_t row_stride_bytes, int32_t page_size, int64_t num_pages, void* kv_a_out,
                                    int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride, const void* q,
                                    int64_t q_stride_t, int64_t q_stride_h, int32_t num_heads, void* q_out,
                                    int64_t q_out_stride_t, int64_t q_out_stride_h, mlahip_stream_t stream);

/* Replaces torch_npu.npu_rotary_mul as the indexer calls it (v1/layers/attention/npu_dsa.py:120, 130): the
 * half-rotation pairing, element i with element i + 32, out = cat(x1*c - x2*s, x2*c + x1*s) with x = cat(x1, x2)
 * (the neox branch of layers/rotary_embedding/rotary_embedding_torch_npu.py:146-163).  x [T, N, 64] through its
 * strides -> out [T, N, 64]; entry i*cos_step of a table row belongs to pair i; rows 8-byte aligned; in place is fine. */
int mla_rotary_mul(const void* x, int64_t x_stride_t, int64_t x_stride_h, int64_t num_tokens, int32_t num_heads,
                   const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step, void* out,
                   int64_t out_stride_t, int64_t out_stride_h, mlahip_stream_t stream);

/* ---- absorbed-MLA paged decode ----------------------------------------------------------
 * Replaces the decode call of torch.ops.npu.npu_fused_infer_attention_score, attention/backends/mla.py:781-804
 * (input_layout "TND_NTD", block_size 128, sparse_mode 3): sequence b owns query tokens
 * [b*max_q_len, (b+1)*max_q_len) or [qsl[b], qsl[b+1]); token i of its s tokens sees keys [0, L_b - s + i].
 * `out` is addressed as [T, N, 512] through its strides, so the reference's head-major [N,T,512] result is
 * out_stride_t = 512, out_stride_h = T*512.  Page size is 128.
 * mla_decode_bf16 = mla_decode_bf16_split followed by mla_splitkv_reduce (the N-way merge of
 * attention/ops.py:109-141).  The split phase cuts the 32-token blocks of ALL sequences, laid end to end, into
 * batch * num_splits chunks of equal size, one workgroup each, so ragged sequence lengths do not unbalance the
 * launch; a chunk writes one normalised fp16 partial + fp32 log-sum-exp per sequence it touches.  The workspace
 * therefore holds batch * (num_splits + 1) partials of max_q_len * num_heads rows.  Nothing in the plan is read
 * back to the host: both phases derive it from seq_lens on the device. */
size_t mla_decode_workspace_bytes(int32_t batch, int32_t max_q_len, int32_t num_heads, int32_t num_splits);

int mla_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h,   /* bf16 [T,N,512] */
                    const void* q_rope, int64_t qr_stride_t, int64_t qr_stride_h,   /* bf16 [T,N,64]  */
                    const void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride,
                    const void* rope_cache, int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                    const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                    const int32_t* seq_lens, const int32_t* query_start_loc /* may be NULL */,
                    int32_t batch, int32_t max_q_len, int32_t num_heads, float scale,
                    void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out /* fp32 [T,N] or NULL */,
                    void* workspace, size_t workspace_bytes, int32_t num_splits, mlahip_stream_t stream);

/* A whole decode step in two launches: the cache write of the step's new tokens (the reshape-and-cache the reference
 * runs in front of its decode, attention/backends/mla.py:868-881) rides in the split kernel, then the merge.  Token t
 * (query_start_loc order, or b * max_q_len + j) brings latent row new_c[t] and rope row new_r[t] for cache row
 * slot_mapping[t]; negative slots are skipped.  The row of key position p of sequence b is stored by the workgroup
 * whose chunk holds p, before that workgroup reads any key: the result equals mla_cache_write_bf16 followed by
 * mla_decode_bf16 for every sequence whose seq_lens counts its new tokens.  (Rows of a request with fewer cached keys
 * than query tokens - an empty padding request - are not written.)  Page size 128.  With out == NULL only the first
 * launch runs and the partials stay in the workspace for mla_splitkv_reduce. */
int mla_decode_bf16_step(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                         int64_t qr_stride_t, int64_t qr_stride_h, void* nope_cache, int64_t nope_page_stride,
                         int64_t nope_row_stride, void* rope_cache, int64_t rope_page_stride, int64_t rope_row_stride,
                         int64_t num_pages, const void* new_c /* bf16 [T,512] */, int64_t new_c_stride,
                         const void* new_r /* bf16 [T,64] */, int64_t new_r_stride, const int64_t* slot_mapping,
                         const int32_t* block_table, int64_t bt_stride, int32_t max_blocks, const int32_t* seq_lens,
                         const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                         float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out,
                         void* workspace, size_t workspace_bytes, int32_t num_splits, mlahip_stream_t stream);

/* The same decode without a workspace argument, for callers that cannot allocate or hand one over: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  (No counterpart in the reference: its vendor op
 * owns its scratch.)  The split-KV partials live in a device array built into the library,
 * MLA_DECODE_STATIC_SCRATCH_BYTES per GPU, held until the process ends; a shape that needs more
 * (mla_decode_workspace_bytes) is refused with -4.  The call allocates and frees nothing.  Calls that overlap in time
 * on one GPU share the array and race: keep them on one stream or order them with events.
 * The FIRST call on each device must run outside stream capture: it looks the array's address up (which makes the
 * runtime load the code object that holds the array) and raises the dynamic LDS limit of the split kernel in all its
 * forms, neither of which may be recorded into a graph.  Every later call, of any shape, only launches kernels and can
 * be captured.  The array is part of the
 * library's image: every process that loads the library pays the 48 MiB on each GPU it touches, whether or not it
 * ever calls this entry point. */
#define MLA_DECODE_STATIC_SCRATCH_BYTES ((size_t)48 << 20)
int mla_decode_bf16_static(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                           int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache, int64_t nope_page_stride,
                           int64_t nope_row_stride, const void* rope_cache, int64_t rope_page_stride,
                           int64_t rope_row_stride, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                           int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                           int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                           int64_t out_stride_h, float* lse_out, int32_t num_splits, mlahip_stream_t stream);

int mla_decode_bf16_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                          int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache, int64_t nope_page_stride,
                          int64_t nope_row_stride, const void* rope_cache, int64_t rope_page_stride,
                          int64_t rope_row_stride, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                          int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                          int32_t max_q_len, int32_t num_heads, float scale, void* workspace, size_t workspace_bytes,
                          int32_t num_splits, mlahip_stream_t stream);

/* seq_lens: the array the split phase was given (the partials are in its chunk order; required).  Output rows must be 16-byte aligned (strides multiples of 8 elements). */
int mla_splitkv_reduce(const void* workspace, size_t workspace_bytes, const int32_t* seq_lens,
                       const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                       int32_t num_splits, void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out,
                       mlahip_stream_t stream);

/* mla_splitkv_reduce with the value up-projection of attention/backends/mla.py:309-315 (_v_up_proj; DSA:
 * dsa.py:233-240) fused in: out[t, n, v] = sum_c o[t, n, c] * w_uv[n, c, v] for the num_tokens query tokens, o being
 * the merged (bf16-rounded) attention result that mla_splitkv_reduce would have written.  w_uv is the reference's
 * W_UV, bf16 [N, 512, 128] through (w_stride_n, w_stride_k) in elements, last dim contiguous; `out` is addressed as
 * [T, N, 128] through its strides (the reference's [T, N*128] output is out_stride_t = N*128, out_stride_h = 128).
 * Replaces four launches of the reference's sequence (merge, batched GEMM, transpose, copy into the output). */
int mla_splitkv_reduce_vup(const void* workspace, size_t workspace_bytes, const int32_t* seq_lens,
                           const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                           int32_t num_splits, int32_t num_tokens, const void* w_uv, int64_t w_stride_n,
                           int64_t w_stride_k, void* out, int64_t out_stride_t, int64_t out_stride_h,
                           mlahip_stream_t stream);

/* Same decode over the fp8-e4m3 block-scaled cache written by mla_cache_write_fp8 (row stride exactly 656 bytes,
 * page size 128).  Tiles are dequantised to bf16 on chip and take the bf16 MFMA path ("dequantise, then attend").
 * No reference counterpart: attention/backends/mla.py:791-792 passes antiquant_mode=0, antiquant_scale=None.
 * out == NULL runs the split phase only: the partials stay in the workspace for mla_splitkv_reduce or
 * mla_splitkv_reduce_vup (same seq_lens / query_start_loc / batch / max_q_len / num_heads / num_splits). */
int mla_decode_fp8(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope, int64_t qr_stride_t,
                   int64_t qr_stride_h, const void* cache, int64_t page_stride_bytes, int64_t row_stride_bytes,
                   int64_t num_pages, const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                   const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch, int32_t max_q_len,
                   int32_t num_heads, float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out,
                   void* workspace, size_t workspace_bytes, int32_t num_splits, mlahip_stream_t stream);

/* ---- chunked-context helpers -------------------------------------------------------------
 * mla_gather_paged replaces ops.gather_and_maybe_dequant_cache (attention/ops.py:5-41, which never dequantises):
 * dst[cu[i] + j] = cat(nope[row], rope[row]) for position seq_starts[i] + j, j < cu[i+1]-cu[i].
 * mla_merge_states replaces ops.merge_attn_states (attention/ops.py:44-106): +inf lse reads as -inf, both sides
 * empty gives zeros and -inf.  dtype codes: 0 = bf16, 1 = fp32. */
int mla_gather_paged(const void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                     int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages, int32_t page_size, void* dst,
                     int64_t dst_row_stride, int64_t dst_rows, const int32_t* block_table, int64_t bt_stride,
                     int32_t max_blocks, const int32_t* cu_seq_lens, const int32_t* seq_starts /* may be NULL */,
                     int32_t batch, int64_t total_rows_hint, mlahip_stream_t stream);

/* The same gather out of the fp8 block-scaled cache (rows of 656 bytes, see mla_cache_write_fp8): the latent part is
 * dequantised to bf16 (e4m3 x block scale, rounded once), the rope part copied.  The reference's
 * gather_and_maybe_dequant_cache (attention/ops.py:5-41) takes kv_cache_dtype and a scale for this case and ignores
 * them; the chunked-context prefill (attention/backends/mla.py:377-450) needs the dequantised rows. */
int mla_gather_paged_fp8(const void* cache, int64_t page_stride_bytes, int64_t row_stride_bytes, int64_t num_pages,
                         int32_t page_size, void* dst, int64_t dst_row_stride, int64_t dst_rows,
                         const int32_t* block_table, int64_t bt_stride, int32_t max_blocks, const int32_t* cu_seq_lens,
                         const int32_t* seq_starts /* may be NULL */, int32_t batch, int64_t total_rows_hint,
                         mlahip_stream_t stream);

int mla_merge_states(const void* prefix_out, int64_t po_stride_t, int64_t po_stride_h, const float* prefix_lse,
                     const void* suffix_out, int64_t so_stride_t, int64_t so_stride_h, const float* suffix_lse,
                     int32_t in_dtype, void* out, int64_t out_stride_t, int64_t out_stride_h, int32_t out_dtype,
                     float* out_lse /* may be NULL */, int32_t tokens, int32_t heads, int32_t dim, mlahip_stream_t stream);

/* N-way merge: replaces attention_update_torch (attention/ops.py:109-141), the torch stand-in of
 * torch_npu.npu_attention_update: outs [n, T, D] (dtype code 0 = bf16, 1 = fp32, 2 = fp16; last dimension contiguous),
 * lses fp32 [n, T] -> out fp32 [T, D], lse_out fp32 [T] (may be NULL).  +inf log-sum-exps read as -inf; a row whose
 * partials all weigh nothing gives zeros and -inf.  One launch for any n. */
int mla_merge_n_states(const void* outs, int64_t outs_stride_n, int64_t outs_stride_t, int32_t in_dtype, const float* lses,
                       int64_t lses_stride_n, float* out, int64_t out_stride_t, float* lse_out, int32_t n, int32_t tokens,
                       int32_t dim, mlahip_stream_t stream);

/* ---- non-absorbed varlen attention for prefill -------------------------------------------
 * Replaces the prefill calls of npu_fused_infer_attention_score, attention/backends/mla.py:574-590 (suffix:
 * right-down causal, sparse_mode 3) and :415-431 (context chunk: no mask, softmax_lse_flag): q_nope [T,N,128],
 * q_pe [T,N,64], k_nope [Tk,N,128], k_pe [Tk,64] shared by all heads (mla.py:579 repeats it), v [Tk,N,128];
 * cu_q / cu_k int32 [B+1] on the device; out [T,N,128] bf16 (0) or fp32 (1); lse_out fp32 [T,N] or NULL.
 * window = w > 0 keeps only the newest w visible keys of each row: the band of mla.py:525-541 (sparse_mode 4,
 * pre_tokens = sliding_window - 1, next_tokens 0); 0 = no window.
 * Rows with no visible key give zeros and lse = -inf.
 * out_dtype + MLA_PREFILL_KV_F16: k_nope, k_pe and v hold fp16 instead of bf16 (a caller that makes them with an fp16
 * GEMM; the queries stay bf16).  Both products then run on fp16 and the kernel skips the bf16 -> fp16 conversion of the value
 * tiles that it otherwise does for the P.V product. */
#define MLA_PREFILL_KV_F16 16
int mla_prefill_varlen(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_pe,
                       int64_t qp_stride_t, int64_t qp_stride_h, const void* k_nope, int64_t kn_stride_t,
                       int64_t kn_stride_h, const void* k_pe, int64_t kp_stride_t, const void* v, int64_t v_stride_t,
                       int64_t v_stride_h, const int32_t* cu_q, const int32_t* cu_k, int32_t batch, int32_t num_heads,
                       int32_t max_q_len, int32_t causal, int32_t window, float scale, void* out, int64_t out_stride_t,
                       int64_t out_stride_h, int32_t out_dtype, float* lse_out, mlahip_stream_t stream);

/* The same attention continued from an earlier result over OTHER keys of the same rows: prev_out fp32 [T,N,128] (strides
 * in elements) and prev_lse fp32 [T,N] contiguous are what an earlier call returned (out_dtype 1, lse_out); the call returns
 * the attention over the union of both key sets.  Replaces the pair "FIA over a context chunk, then merge_attn_states"
 * of the reference's chunked-context loop (attention/backends/mla.py:415-447 with attention/ops.py:5-42) and the final
 * merge of context and suffix (mla.py:594-606) by one launch each.  Rows whose prev_lse is -inf or +inf start empty, as
 * the reference's merge treats them.  out may be prev_out and lse_out may be prev_lse. */
int mla_prefill_varlen_continue(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_pe,
                                int64_t qp_stride_t, int64_t qp_stride_h, const void* k_nope, int64_t kn_stride_t,
                                int64_t kn_stride_h, const void* k_pe, int64_t kp_stride_t, const void* v,
                                int64_t v_stride_t, int64_t v_stride_h, const int32_t* cu_q, const int32_t* cu_k,
                                int32_t batch, int32_t num_heads, int32_t max_q_len, int32_t causal, int32_t window,
                                float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, int32_t out_dtype,
                                float* lse_out, const float* prev_out, int64_t prev_stride_t, int64_t prev_stride_h,
                                const float* prev_lse, mlahip_stream_t stream);

/* ---- DSA lightning indexer --------------------------------------------------------------------
 * Replaces torch.ops.custom.npu_lightning_indexer, v1/layers/attention/npu_dsa.py:92-103 and
 * vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:133-146, in two steps:
 * dsa_indexer_scores_fp8: logits[t,s] = k_scale[s] * sum_h w[t,h] (* q_scale[t,h]) * relu(q8[t,h,:] . k8[s,:])
 * for the visible keys s of token t (64 heads, 128-wide float8_e4m3fn rows, fp32 scales; pages hold a multiple of 32 keys,
 * key rows lie 128 .. 2^20 bytes apart, the scales of a page are contiguous);
 * dsa_topk: positions of the k largest logits, ties to the lower position, ascending order, -1 padding
 * (int32 [T,k], the reference's [T,1,topk] buffer). */
int dsa_indexer_scores_fp8(const void* q8, int64_t q_stride_t, int64_t q_stride_h, const float* weights,
                           int64_t w_stride_t, const float* q_scale /* may be NULL */, int64_t qs_stride_t,
                           const void* k8_cache, int64_t k_page_stride, int64_t k_row_stride, const float* k_scale_cache,
                           int64_t ks_page_stride, int64_t num_pages, int32_t page_size, const int32_t* block_table,
                           int64_t bt_stride, int32_t max_blocks, const int32_t* seq_lens,
                           const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                           int32_t max_seq_len, float* logits, int64_t logits_stride, mlahip_stream_t stream);

/* Per-row e4m3 quantisation of 128-wide bf16 rows (scale = amax/448 per row), optionally scattered through a slot
 * mapping into the paged fp8 indexer-K cache and its scale cache: the indexer-K scatter of patch_dsv32_indexer.py:116-121
 * with the quantisation fused in; with slot_mapping == NULL it quantises the query rows in place order. */
int dsa_quant_rows_fp8(const void* src, int64_t src_stride, int64_t rows, const int64_t* slot_mapping /* may be NULL */,
                       void* dst8, int64_t dst_page_stride_bytes, int64_t dst_row_stride_bytes, float* dst_scale,
                       int64_t scale_page_stride, int32_t page_size, int64_t num_pages, mlahip_stream_t stream);

/* dsa_quant_rows_fp8 twice in one launch, the way the indexer needs it every step (patch_dsv32_indexer.py:116-131: the new
 * index keys go into the cache, the queries are handed to the scoring op): q rows [q_rows, 128] -> q8 [q_rows, 128] +
 * q_scale [q_rows]; k rows [k_rows, 128] -> row slot_mapping[r] of the paged key cache and of its scale plane. */
int dsa_quant_qk_fp8(const void* q, int64_t q_stride, int64_t q_rows, void* q8, float* q_scale, const void* k,
                     int64_t k_stride, int64_t k_rows, const int64_t* slot_mapping, void* k8_cache,
                     int64_t cache_page_stride_bytes, int64_t cache_row_stride_bytes, float* scale_cache,
                     int64_t scale_page_stride, int32_t page_size, int64_t num_pages, mlahip_stream_t stream);

/* With a workspace of dsa_topk_workspace_bytes() the selection of a token is spread over several workgroups (three
 * launches that meet in the workspace: slice histograms, boundary-bin gather, ordered write), which is what a
 * decode step with few tokens and long rows needs; with workspace == NULL one workgroup per token does everything and
 * no scratch memory is touched.  Both give identical results. */
size_t dsa_topk_workspace_bytes(int32_t batch, int32_t max_q_len, int64_t logits_stride);
int dsa_topk(const float* logits, int64_t logits_stride, const int32_t* seq_lens, const int32_t* query_start_loc,
             int32_t batch, int32_t max_q_len, int32_t k, int32_t* out_indices, int64_t out_stride,
             void* workspace /* may be NULL */, size_t workspace_bytes, mlahip_stream_t stream);

/* dsa_topk and dsa_build_rows (below) in one pass: besides the positions every pick is translated through the block
 * table into its flat cache row (page * page_size + offset) and counts[t] = picks of token t; what
 * attention/backends/dsa.py:259-291 feeds to the sparse attention, without a second launch. */
int dsa_topk_rows(const float* logits, int64_t logits_stride, const int32_t* seq_lens, const int32_t* query_start_loc,
                  int32_t batch, int32_t max_q_len, int32_t k, int32_t* out_indices, int64_t out_stride,
                  const int32_t* block_table, int64_t bt_stride, int32_t max_blocks, int32_t page_size, int64_t num_pages,
                  int32_t* rows, int64_t rows_stride, int32_t* counts, void* workspace /* may be NULL */,
                  size_t workspace_bytes, mlahip_stream_t stream);

/* ---- sparse MLA over the selected keys ----------------------------------------------------------
 * Replaces torch.ops.custom.npu_sparse_flash_attention, attention/backends/dsa.py:259-291 (sparse_block_size 1,
 * layout_kv "PA_BSND"): dsa_build_rows maps the [T,k] logical positions (-1 = unused,
 * v1/layers/attention/npu_dsa.py:553-555) through the block table to flat cache rows, compacted, with a count per
 * token; dsa_sparse_decode_bf16 runs the absorbed-MLA kernel over those rows (cache pages must be contiguous).
 * out == NULL runs its split phase only; the merge is then mla_splitkv_reduce or mla_splitkv_reduce_vup with
 * seq_lens = counts, query_start_loc = NULL, batch = num_tokens, max_q_len = 1. */
int dsa_build_rows(const int32_t* indices, int64_t indices_stride, const int32_t* block_table, int64_t bt_stride,
                   int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                   int32_t max_q_len, int32_t k, int32_t page_size, int64_t num_pages, int32_t* rows,
                   int64_t rows_stride, int32_t* counts, mlahip_stream_t stream);

/* Decode with static sink tokens and a sliding window on the dense kernel (attention/backends/mla.py:705-779: the
 * reference runs one attention over the sink pages, one over the last sliding_window keys behind them and merges the two
 * by LSE; this is the same softmax over the union of the keys in one pass).  The first sink_len / 128 pages of every
 * block-table row hold the sink keys; seq_lens counts the keys behind them; token i of a request with s query tokens
 * sees the sink and keys [max(0, L - s + i + 1 - window), L - s + i] behind it.
 * mla_window_plan writes, per sequence, the number of 32-key blocks between the sink and the oldest visible key (skip)
 * and the length of the sequence without them (short_lens); mla_decode_bf16_window_split is mla_decode_bf16_split over
 * those shortened sequences; the merge is mla_splitkv_reduce / mla_splitkv_reduce_vup with seq_lens = short_lens. */
int mla_window_plan(const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch, int32_t max_q_len,
                    int32_t sink_len, int32_t window, int32_t* short_lens, int32_t* skip, mlahip_stream_t stream);

int mla_decode_bf16_window_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                 int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache, int64_t nope_page_stride,
                                 int64_t nope_row_stride, const void* rope_cache, int64_t rope_page_stride,
                                 int64_t rope_row_stride, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                                 int32_t max_blocks, const int32_t* short_lens, const int32_t* skip,
                                 const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                 int32_t sink_len, int32_t window, float scale, void* workspace, size_t workspace_bytes,
                                 int32_t num_splits, mlahip_stream_t stream);

/* The same split phase over the fp8 block-scaled cache of mla_decode_fp8 (no counterpart call in the reference, which has
 * no fp8 latent cache; the variant is the one of mla.py:705-779). */
int mla_decode_fp8_window_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                int64_t qr_stride_t, int64_t qr_stride_h, const void* cache, int64_t page_stride_bytes,
                                int64_t row_stride_bytes, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                                int32_t max_blocks, const int32_t* short_lens, const int32_t* skip,
                                const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                int32_t sink_len, int32_t window, float scale, void* workspace, size_t workspace_bytes,
                                int32_t num_splits, mlahip_stream_t stream);

int dsa_sparse_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                           int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache, int64_t nope_page_stride,
                           int64_t nope_row_stride, const void* rope_cache, int64_t rope_page_stride,
                           int64_t rope_row_stride, int64_t num_pages, int32_t page_size, const int32_t* sparse_rows,
                           int64_t sparse_stride, const int32_t* counts, int32_t num_tokens, int32_t num_heads,
                           float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out,
                           void* workspace, size_t workspace_bytes, int32_t num_splits, mlahip_stream_t stream);

/* The same sparse attention with the work split over HEADS instead of keys: a workgroup owns (token, 16 heads), walks all
 * of the token's rows and writes the bf16 result itself - one launch, no workspace, nothing to merge (the form for many
 * heads and a few thousand selected keys per token: attention/backends/dsa.py:259-291 at decode).  num_heads a multiple
 * of 16; the caches are addressed as flat rows (num_rows of them, row strides in elements), i.e. pages must be contiguous. */
int dsa_sparse_decode_heads_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                 int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache, int64_t nope_row_stride,
                                 const void* rope_cache, int64_t rope_row_stride, int64_t num_rows,
                                 const int32_t* sparse_rows, int64_t sparse_stride, const int32_t* counts,
                                 int32_t num_tokens, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                                 int64_t out_stride_h, float* lse_out /* fp32 [T,N] or NULL */, mlahip_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MLA_HIP_H */
