// Paged gather of latent rows into a contiguous workspace, and the two-way log-sum-exp merge of
// attention states: the two torch helpers of the reference's chunked-context prefill,
// src/omni_npu/attention/ops.py:5-41 (gather_and_maybe_dequant_cache, which never dequantises) and
// ops.py:44-106 (merge_attn_states).
#include "mla_common.hpp"

namespace mlahip {

// One wavefront per destination row: dst[cu[i] + j] = cat(nope[row], rope[row]) for position seq_starts[i] + j.
__global__ __launch_bounds__(256) void gather_paged_kernel(const char* nope, int64_t nope_sp, int64_t nope_sr,
                                                           const char* rope, int64_t rope_sp, int64_t rope_sr,
                                                           char* dst, int64_t dst_stride_b, const int32_t* block_table,
                                                           int64_t bt_stride, int32_t max_blocks, const int32_t* cu_seq_lens,
                                                           const int32_t* seq_starts, int32_t batch, int32_t page_size,
                                                           int64_t num_pages, int64_t dst_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t total = cu_seq_lens[batch];
  if (row >= total || row >= dst_rows) return;
  int lo = 0, hi = batch;                          // largest i with cu[i] <= row
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_seq_lens[mid] <= row) lo = mid; else hi = mid;
  }
  const int64_t pos = (seq_starts ? seq_starts[lo] : 0) + (row - cu_seq_lens[lo]);
  int64_t pg = pos / page_size;
  const int64_t off = pos - pg * page_size;
  pg = pg < max_blocks ? pg : max_blocks - 1;
  int64_t blk = block_table[(int64_t)lo * bt_stride + pg];
  blk = blk < 0 ? 0 : (blk >= num_pages ? num_pages - 1 : blk);
  char* d = dst + row * dst_stride_b;
  *(u32x4*)(d + lane * 16) = *(const u32x4*)(nope + blk * nope_sp + off * nope_sr + lane * 16);
  if (lane < 8) *(u32x4*)(d + kDNope * 2 + lane * 16) = *(const u32x4*)(rope + blk * rope_sp + off * rope_sr + lane * 16);
}

// The same gather out of the fp8 block-scaled cache (rows of 512 e4m3 | 4 fp32 scales | 64 bf16 rope, see
// cache_write_fp8_kernel): dst row = cat(bf16(e4m3 * block scale), rope), the values the fp8 decode kernel attends over.
__global__ __launch_bounds__(256) void gather_paged_fp8_kernel(const char* cache, int64_t page_stride_b, int64_t row_stride_b,
                                                               char* dst, int64_t dst_stride_b, const int32_t* block_table,
                                                               int64_t bt_stride, int32_t max_blocks,
                                                               const int32_t* cu_seq_lens, const int32_t* seq_starts,
                                                               int32_t batch, int32_t page_size, int64_t num_pages,
                                                               int64_t dst_rows) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t total = cu_seq_lens[batch];
  if (row >= total || row >= dst_rows) return;
  int lo = 0, hi = batch;                          // largest i with cu[i] <= row
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_seq_lens[mid] <= row) lo = mid; else hi = mid;
  }
  const int64_t pos = (seq_starts ? seq_starts[lo] : 0) + (row - cu_seq_lens[lo]);
  int64_t pg = pos / page_size;
  const int64_t off = pos - pg * page_size;
  pg = pg < max_blocks ? pg : max_blocks - 1;
  int64_t blk = block_table[(int64_t)lo * bt_stride + pg];
  blk = blk < 0 ? 0 : (blk >= num_pages ? num_pages - 1 : blk);
  const char* src = cache + blk * page_stride_b + off * row_stride_b;
  char* d = dst + row * dst_stride_b;
  const u32x2 q = *(const u32x2*)(src + lane * 8);               // eight e4m3 values
  const float scale = *(const float*)(src + 512 + (lane >> 4) * 4);   // one scale per 128 elements = 16 lanes
  bf16x8 o;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const f32x2 lo2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[h], false), hi2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)q[h], true);
    o[4 * h + 0] = (__bf16)(lo2[0] * scale);
    o[4 * h + 1] = (__bf16)(lo2[1] * scale);
    o[4 * h + 2] = (__bf16)(hi2[0] * scale);
    o[4 * h + 3] = (__bf16)(hi2[1] * scale);
  }
  *(bf16x8*)(d + lane * 16) = o;
  if (lane < 8) *(u32x4*)(d + kDNope * 2 + lane * 16) = *(const u32x4*)(src + 528 + lane * 16);
}

template <typename T> __device__ __forceinline__ float ld(const T* p) { return (float)*p; }
template <typename T> __device__ __forceinline__ void st(T* p, float v) { *p = (T)v; }

// One wavefront per (token, head) row of width D.
template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void merge_states_kernel(const TIn* po, int64_t po_st, int64_t po_sh, const float* pl,
                                                           const TIn* so, int64_t so_st, int64_t so_sh, const float* sl,
                                                           TOut* out, int64_t out_st, int64_t out_sh, float* out_lse,
                                                           int32_t tokens, int32_t heads, int32_t dim) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= (int64_t)tokens * heads) return;
  const int64_t t = r / heads, h = r - t * heads;
  float a = pl[r], b = sl[r];
  a = a == INFINITY ? -INFINITY : a;               // +inf is what some kernels report for empty rows
  b = b == INFINITY ? -INFINITY : b;
  const float m = fmaxf(a, b);
  float wa = 0.f, wb = 0.f, lse = -INFINITY;
  if (m != -INFINITY) {
    const float ea = __expf(a - m), eb = __expf(b - m);
    const float tot = ea + eb;
    wa = ea / tot;
    wb = eb / tot;
    lse = __logf(tot) + m;
  }
  const TIn* p = po + t * po_st + h * po_sh;
  const TIn* s = so + t * so_st + h * so_sh;
  TOut* o = out + t * out_st + h * out_sh;
  for (int i = lane; i < dim; i += 64) {
    // a side with zero weight contributes nothing even if it holds NaN / inf garbage
    const float pv = wa > 0.f ? ld(p + i) * wa : 0.f;
    const float sv = wb > 0.f ? ld(s + i) * wb : 0.f;
    st(o + i, pv + sv);
  }
  if (out_lse && lane == 0) out_lse[r] = lse;
}

// N-way merge of attention partials (src/omni_npu/attention/ops.py:109-141): outs [n, T, D], lses [n, T] ->
// out fp32 [T, D], lse fp32 [T].  +inf log-sum-exps read as -inf; a row whose partials all weigh nothing gives zeros
// and -inf; a partial with zero weight contributes nothing even if it holds NaN / inf garbage.  One wavefront per row:
// the weights are worked out once (lane p holds partial p, up to 64 at a time), then the lanes walk the row's columns.
template <typename TIn>
__global__ __launch_bounds__(256) void merge_n_states_kernel(const TIn* __restrict__ outs, int64_t o_sn, int64_t o_st,
                                                            const float* __restrict__ lses, int64_t l_sn,
                                                            float* __restrict__ out, int64_t out_st, float* __restrict__ lse_out,
                                                            int32_t n, int32_t tokens, int32_t dim) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= tokens) return;
  auto lse_of = [&](int q) -> float {
    float l = q < n ? lses[(int64_t)q * l_sn + t] : -INFINITY;
    return l == INFINITY ? -INFINITY : l;
  };
  float m = -INFINITY;
  for (int q0 = 0; q0 < n; q0 += 64) m = fmaxf(m, lse_of(q0 + lane));
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
  float se = 0.f;
  if (m != -INFINITY)
    for (int q0 = 0; q0 < n; q0 += 64) se += __expf(lse_of(q0 + lane) - m);
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) se += __shfl_xor(se, d, 64);
  const bool valid = se > 0.f;                              // (false also for NaN)
  for (int i = lane; i < dim; i += 64) {
    float a = 0.f;
    if (valid)
      for (int q = 0; q < n; q++) {
        const float w = __expf(lse_of(q) - m) / se;
        if (w > 0.f) a += ld(outs + (int64_t)q * o_sn + t * o_st + i) * w;
      }
    out[t * out_st + i] = a;
  }
  if (lse_out && lane == 0) lse_out[t] = valid ? __logf(se) + m : -INFINITY;
}

}  // namespace mlahip
using namespace mlahip;

// dtype codes: 0 = bf16, 1 = fp32, 2 = fp16
extern "C" int mla_merge_n_states(const void* outs, int64_t outs_stride_n, int64_t outs_stride_t, int32_t in_dtype,
                                  const float* lses, int64_t lses_stride_n, float* out, int64_t out_stride_t, float* lse_out,
                                  int32_t n, int32_t tokens, int32_t dim, hipStream_t stream) {
  MLA_REQUIRE(outs && lses && out, MLA_ERR_NULL, "mla_merge_n_states: null pointer argument");
  MLA_REQUIRE(n >= 1 && tokens >= 0 && dim >= 1, MLA_ERR_SHAPE, "mla_merge_n_states: n=%d tokens=%d dim=%d", n, tokens, dim);
  MLA_REQUIRE(in_dtype >= 0 && in_dtype <= 2, MLA_ERR_UNSUPPORTED, "mla_merge_n_states: dtype codes are 0 (bf16), 1 (fp32), 2 (fp16)");
  if (tokens == 0) return MLA_OK;
  const dim3 grid((unsigned)(((int64_t)tokens + 3) / 4)), block(256);
#define MLA_MERGE_N(TI)                                                                                                  \
  hipLaunchKernelGGL((merge_n_states_kernel<TI>), grid, block, 0, stream, (const TI*)outs, outs_stride_n, outs_stride_t, \
                     lses, lses_stride_n, out, out_stride_t, lse_out, n, tokens, dim)
  if (in_dtype == 0) MLA_MERGE_N(__bf16);
  else if (in_dtype == 1) MLA_MERGE_N(float);
  else MLA_MERGE_N(_Float16);
#undef MLA_MERGE_N
  return check_launch("mla_merge_n_states");
}

extern "C" int mla_gather_paged(const void* nope_cache, int64_t nope_page_stride, int64_t nope_row_stride,
                                const void* rope_cache, int64_t rope_page_stride, int64_t rope_row_stride,
                                int64_t num_pages, int32_t page_size, void* dst, int64_t dst_row_stride, int64_t dst_rows,
                                const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                const int32_t* cu_seq_lens, const int32_t* seq_starts, int32_t batch,
                                int64_t total_rows_hint, hipStream_t stream) {
  MLA_REQUIRE(nope_cache && rope_cache && dst && block_table && cu_seq_lens, MLA_ERR_NULL,
              "mla_gather_paged: null pointer argument");
  MLA_REQUIRE(batch >= 0 && page_size >= 1 && num_pages >= 1 && max_blocks >= 1 && dst_rows >= 0 && total_rows_hint >= 0,
              MLA_ERR_SHAPE, "mla_gather_paged: batch=%d page_size=%d num_pages=%lld max_blocks=%d", batch, page_size,
              (long long)num_pages, max_blocks);
  MLA_REQUIRE(nope_row_stride % 8 == 0 && rope_row_stride % 8 == 0 && nope_page_stride % 8 == 0 &&
                  rope_page_stride % 8 == 0 && dst_row_stride % 8 == 0 && dst_row_stride >= kDNope + kDRope &&
                  (uintptr_t)nope_cache % 16 == 0 && (uintptr_t)rope_cache % 16 == 0 && (uintptr_t)dst % 16 == 0,
              MLA_ERR_SHAPE, "mla_gather_paged: rows must be 16-byte aligned and dst rows at least 576 wide");
  const int64_t rows = total_rows_hint < dst_rows ? total_rows_hint : dst_rows;
  if (batch == 0 || rows == 0) return MLA_OK;
  hipLaunchKernelGGL(gather_paged_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, (const char*)nope_cache,
                     nope_page_stride * 2, nope_row_stride * 2, (const char*)rope_cache, rope_page_stride * 2,
                     rope_row_stride * 2, (char*)dst, dst_row_stride * 2, block_table, bt_stride, max_blocks, cu_seq_lens,
                     seq_starts, batch, page_size, num_pages, dst_rows);
  return check_launch("mla_gather_paged");
}

extern "C" int mla_gather_paged_fp8(const void* cache, int64_t page_stride_bytes, int64_t row_stride_bytes, int64_t num_pages,
                                    int32_t page_size, void* dst, int64_t dst_row_stride, int64_t dst_rows,
                                    const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                    const int32_t* cu_seq_lens, const int32_t* seq_starts, int32_t batch,
                                    int64_t total_rows_hint, hipStream_t stream) {
  MLA_REQUIRE(cache && dst && block_table && cu_seq_lens, MLA_ERR_NULL, "mla_gather_paged_fp8: null pointer argument");
  MLA_REQUIRE(batch >= 0 && page_size >= 1 && num_pages >= 1 && max_blocks >= 1 && dst_rows >= 0 && total_rows_hint >= 0,
              MLA_ERR_SHAPE, "mla_gather_paged_fp8: batch=%d page_size=%d num_pages=%lld max_blocks=%d", batch, page_size,
              (long long)num_pages, max_blocks);
  MLA_REQUIRE(row_stride_bytes >= 656 && row_stride_bytes % 16 == 0 && page_stride_bytes % 16 == 0 && dst_row_stride % 8 == 0 &&
                  dst_row_stride >= kDNope + kDRope && (uintptr_t)cache % 16 == 0 && (uintptr_t)dst % 16 == 0,
              MLA_ERR_SHAPE, "mla_gather_paged_fp8: cache rows are 656 bytes, 16-byte aligned; dst rows at least 576 wide");
  const int64_t rows = total_rows_hint < dst_rows ? total_rows_hint : dst_rows;
  if (batch == 0 || rows == 0) return MLA_OK;
  hipLaunchKernelGGL(gather_paged_fp8_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, (const char*)cache,
                     page_stride_bytes, row_stride_bytes, (char*)dst, dst_row_stride * 2, block_table, bt_stride, max_blocks,
                     cu_seq_lens, seq_starts, batch, page_size, num_pages, dst_rows);
  return check_launch("mla_gather_paged_fp8");
}

// dtype codes: 0 = bf16, 1 = fp32
extern "C" int mla_merge_states(const void* prefix_out, int64_t po_stride_t, int64_t po_stride_h, const float* prefix_lse,
                                const void* suffix_out, int64_t so_stride_t, int64_t so_stride_h, const float* suffix_lse,
                                int32_t in_dtype, void* out, int64_t out_stride_t, int64_t out_stride_h, int32_t out_dtype,
                                float* out_lse, int32_t tokens, int32_t heads, int32_t dim, hipStream_t stream) {
  MLA_REQUIRE(prefix_out && prefix_lse && suffix_out && suffix_lse && out, MLA_ERR_NULL,
              "mla_merge_states: null pointer argument");
  MLA_REQUIRE(tokens >= 0 && heads >= 1 && dim >= 1, MLA_ERR_SHAPE, "mla_merge_states: tokens=%d heads=%d dim=%d", tokens,
              heads, dim);
  MLA_REQUIRE((in_dtype == 0 || in_dtype == 1) && (out_dtype == 0 || out_dtype == 1), MLA_ERR_UNSUPPORTED,
              "mla_merge_states: dtype codes are 0 (bf16) and 1 (fp32)");
  if (tokens == 0) return MLA_OK;
  const dim3 grid((unsigned)(((int64_t)tokens * heads + 3) / 4)), block(256);
#define MLA_MERGE(TI, TO)                                                                                              \
  hipLaunchKernelGGL((merge_states_kernel<TI, TO>), grid, block, 0, stream, (const TI*)prefix_out, po_stride_t,        \
                     po_stride_h, prefix_lse, (const TI*)suffix_out, so_stride_t, so_stride_h, suffix_lse, (TO*)out,   \
                     out_stride_t, out_stride_h, out_lse, tokens, heads, dim)
  if (in_dtype == 0 && out_dtype == 0) MLA_MERGE(__bf16, __bf16);
  else if (in_dtype == 0 && out_dtype == 1) MLA_MERGE(__bf16, float);
  else if (in_dtype == 1 && out_dtype == 0) MLA_MERGE(float, __bf16);
  else MLA_MERGE(float, float);
#undef MLA_MERGE
  return check_launch("mla_merge_states");
}
