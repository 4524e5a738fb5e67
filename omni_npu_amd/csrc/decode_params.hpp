// Parameters and launchers of the absorbed-MLA split-KV decode kernels (decode_v3.hip, decode_v3_fp8.hip), of the merge
// of their partials (chunk_reduce.hip) and of the merge fused with the value up-projection (reduce_vup.hip).
#pragma once
#include "mla_common.hpp"

namespace mlahip {

struct DecodeParams {
  const __bf16* q_nope; int64_t qn_st, qn_sh;
  const __bf16* q_rope; int64_t qr_st, qr_sh;
  const __bf16* nope; int64_t nope_sp, nope_sr;
  const __bf16* rope; int64_t rope_sp, rope_sr;
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks;
  const int32_t* seq_lens;
  const int32_t* qsl;
  int32_t batch, max_q_len, num_heads;
  int64_t num_pages;
  float scale_log2;
  _Float16* o_part;              // [chunks + B, R_max, 512] fp16, normalised
  float* lse_part;               // [chunks + B, R_max], natural log
  float* corr_scale;             // [chunks + B, R_max]: (p - bf16(p)) / l of the row's dominant key, or 0
  const __bf16** corr_row;       // [chunks + B, R_max]: that key's latent vector in the cache
  int32_t* seg_ids;              // [B][2]: partial number of the sequence's first / last segment
  const int32_t* sparse_rows; int64_t sparse_stride; int32_t page_size;
  const uint8_t* cache8; int64_t c8_sp;   // fp8 kernel: block-scaled cache, page stride in bytes (rows are 656 bytes apart)
  // Sink + sliding window (dense bf16 kernel only): seq_lens then holds the length of the sequence with the 32-key
  // blocks between the sink and the window taken out, win_skip[b] is how many were taken out, and a key behind the
  // sink is visible to a row only if it is one of the newest win_size keys the row may see.
  const int32_t* win_skip; int32_t win_sink, win_size;
  // The step's cache write folded into the dense kernel (null = the cache already holds the new rows): latent row
  // new_c[t] and rope row new_r[t] of query token t go to cache row new_slots[t] (negative = skip), written by the
  // workgroup whose chunk holds that key, before it copies any block.
  const __bf16* new_c; int64_t new_c_st; const __bf16* new_r; int64_t new_r_st; const int64_t* new_slots;
};

struct ChunkReduceParams {
  const _Float16* o_part; const float* lse_part; const float* corr_scale; const __bf16* const* corr_row;
  const int32_t* seg_ids;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, num_heads, num_chunks;
  __bf16* out; int64_t out_st, out_sh;
  float* lse_out; int64_t lse_st;      // optional [T, N]
};
int launch_chunk_reduce(const ChunkReduceParams& p, hipStream_t stream);

// The chunk plan of the split kernels, as the merge kernels recompute it: work is counted in blocks of kPlanBlk keys,
// and every non-empty sequence costs kPlanSegCost more units of start-up.
constexpr int kPlanBlk = 32;
constexpr int kPlanSegCost = 8;
__device__ __forceinline__ int plan_work_units(int len) { return len > 0 ? (len + kPlanBlk - 1) / kPlanBlk + kPlanSegCost : 0; }

// Merge of the partials fused with the value up-projection (reduce_vup.hip): out[t, n*128 + v] = merged o[t,n,:] . W_UV[n,:,v]
int launch_reduce_vup(const ChunkReduceParams& r, const void* w_uv, int64_t w_stride_n, int64_t w_stride_k,
                      int32_t num_tokens, hipStream_t stream);

// The eight-wavefront kernel over the bf16 cache (decode_v3.hip): dense, row-list (sparse) and, with p.win_skip set, sink +
// window.  Returns 0 or a negative error code.
int launch_decode_v3(const DecodeParams& p, bool sparse, dim3 grid, hipStream_t stream);
// The dynamic-LDS limit of all dense bf16 forms raised on the current device, ahead of a launch under stream capture.
int prepare_decode_v3_dense_forms();
// The same over the fp8 block-scaled cache p.cache8 (decode_v3_fp8.hip): dense and, with p.win_skip set, sink + window.
int launch_decode_v3_fp8(const DecodeParams& p, dim3 grid, hipStream_t stream);

}  // namespace mlahip
