// Exact top-k selection for the DSA indexer, and the index -> cache-row translation for sparse MLA.
//
// Replaces the selection half of torch.ops.custom.npu_lightning_indexer
// (src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:133-146: int32 [T,1,topk]
// logical key positions, -1 for unused slots as in src/omni_npu/v1/layers/attention/npu_dsa.py:553-555).
// Semantics: the k largest logits among the visible keys, ties to the LOWER index; the output lists the
// selected positions in ascending position order followed by -1 padding.
//
// One workgroup of 1024 threads per query token.  A radix select over the 64-bit key
//   (order-preserving image of the fp32 logit) << 32 | ~position
// finds the k-th largest key: three 11/11/10-bit passes over the logit bits, and, only when the
// threshold logit is shared by more keys than are still needed, two more passes over the position bits.
// All keys are distinct, so "key >= threshold" selects exactly k elements.  The final pass gives every
// thread a contiguous slice, scans the per-thread counts once, and writes the positions in order.
#include "mla_common.hpp"

namespace mlahip {

constexpr int kTopkThreads = 1024;
constexpr int kBins = 2048;

__device__ __forceinline__ uint32_t ordered_bits(float x) {
  if (x == 0.f) x = 0.f;                                   // -0 and +0 compare equal: one image for both
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Workgroup-wide: given hist[kBins] (count per digit, larger digit = larger key) and `need` (>= 1, <= total),
// find digit d with  count(digit > d) < need <= count(digit >= d).  Returns d, and the count above it via *above.
__device__ int select_digit(int* hist, int* scratch, int need, int* above) {
  const int tid = threadIdx.x;
  // each thread owns 2 bins taken from the top: bins (kBins-1-2*tid) and (kBins-2-2*tid)
  const int b0 = kBins - 1 - 2 * tid, b1 = b0 - 1;
  const int c0 = hist[b0], c1 = hist[b1];
  int v = c0 + c1;
  // inclusive scan over threads (descending bins)
  const int lane = tid & 63, w = tid >> 6;
  int s = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int n = __shfl_up(s, o, 64);
    if (lane >= o) s += n;
  }
  if (lane == 63) scratch[w] = s;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += scratch[i];
  const int incl = base + s, excl = incl - v;              // keys in bins above this thread's pair: excl
  __syncthreads();
  if (excl < need && need <= incl) {                       // exactly one thread
    if (need <= excl + c0) { scratch[32] = b0; scratch[33] = excl; }
    else { scratch[32] = b1; scratch[33] = excl + c0; }
  }
  __syncthreads();
  const int d = scratch[32];
  *above = scratch[33];
  __syncthreads();
  return d;
}

struct TopkParams {
  const float* logits; int64_t l_st;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, k;
  int32_t* out; int64_t o_st;
};

__global__ __launch_bounds__(kTopkThreads) void dsa_topk_kernel(const TopkParams p) {
  __shared__ int hist[kBins];
  __shared__ int scratch[64];
  const int tid = threadIdx.x;
  const int b = blockIdx.x / p.max_q_len;
  const int ti = blockIdx.x - b * p.max_q_len;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  if (ti >= qlen) return;
  const int t = q0 + ti;
  int n = p.seq_lens[b] - qlen + ti + 1;                   // visible keys
  n = n < 0 ? 0 : n;
  const float* x = p.logits + (int64_t)t * p.l_st;
  int32_t* out = p.out + (int64_t)t * p.o_st;
  const int k = p.k;

  if (n <= k) {                                            // everything is selected
    for (int i = tid; i < k; i += kTopkThreads) out[i] = i < n ? i : -1;
    return;
  }

  // ---- radix select on the logit bits ----
  uint32_t prefix = 0, pmask = 0;
  int need = k;                                            // how many keys are still wanted among the matching ones
  const int shifts[3] = {21, 10, 0};
  const int widths[3] = {11, 11, 10};
  for (int pass = 0; pass < 3; pass++) {
    for (int i = tid; i < kBins; i += kTopkThreads) hist[i] = 0;
    __syncthreads();
    const int sh = shifts[pass];
    const uint32_t dm = (1u << widths[pass]) - 1;
    for (int i = tid; i < n; i += kTopkThreads) {
      const uint32_t u = ordered_bits(x[i]);
      if ((u & pmask) == prefix) atomicAdd(&hist[(u >> sh) & dm], 1);
    }
    __syncthreads();
    int above;
    const int d = select_digit(hist, scratch, need, &above);
    need -= above;
    prefix |= (uint32_t)d << sh;
    pmask |= dm << sh;
  }
  // prefix = threshold logit image; `need` of the keys equal to it are wanted (need >= 1)
  // count the equals; if more than needed, select the lowest positions among them
  uint32_t pos_thresh = 0;                                 // wanted equals: position <= pos_thresh ... computed below
  {
    for (int i = tid; i < kBins; i += kTopkThreads) hist[i] = 0;
    __syncthreads();
    // positions < 2^22: two passes over ~position bits (11 + 11); larger digit of ~pos = lower position
    uint32_t ppre = 0, pm = 0;
    const int psh[2] = {11, 0};
    for (int pass = 0; pass < 2; pass++) {
      if (pass) {
        for (int i = tid; i < kBins; i += kTopkThreads) hist[i] = 0;
        __syncthreads();
      }
      for (int i = tid; i < n; i += kTopkThreads) {
        if (ordered_bits(x[i]) == prefix) {
          const uint32_t ip = (~(uint32_t)i) & 0x3FFFFFu;
          if ((ip & pm) == ppre) atomicAdd(&hist[(ip >> psh[pass]) & 0x7FFu], 1);
        }
      }
      __syncthreads();
      int above;
      const int d = select_digit(hist, scratch, need, &above);
      need -= above;
      ppre |= (uint32_t)d << psh[pass];
      pm |= 0x7FFu << psh[pass];
    }
    pos_thresh = (~ppre) & 0x3FFFFFu;                      // the highest position still taken among the equals
  }

  // ---- ordered output: thread tid owns [tid*per, (tid+1)*per) ----
  const int per = (n + kTopkThreads - 1) / kTopkThreads;
  const int lo = tid * per;
  int hi = lo + per;
  hi = hi < n ? hi : n;
  int cnt = 0;
  for (int i = lo; i < hi; i++) {
    const uint32_t u = ordered_bits(x[i]);
    cnt += (u > prefix) || (u == prefix && (uint32_t)i <= pos_thresh);
  }
  const int lane = tid & 63, w = tid >> 6;
  int s = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(s, o, 64);
    if (lane >= o) s += v;
  }
  if (lane == 63) scratch[w] = s;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += scratch[i];
  int o = base + s - cnt;
  for (int i = lo; i < hi; i++) {
    const uint32_t u = ordered_bits(x[i]);
    if ((u > prefix) || (u == prefix && (uint32_t)i <= pos_thresh)) {
      if (o < k) out[o] = i;
      o++;
    }
  }
}

// Sparse-MLA row list: logical positions -> flat cache rows, dropping -1 / out-of-range entries, order kept.
struct RowsParams {
  const int32_t* indices; int64_t i_st;                    // [T, K]
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, k, page_size;
  int64_t num_pages;
  int32_t* rows; int64_t r_st;                             // [T, K] flat rows (page * page_size + offset)
  int32_t* counts;                                         // [T]
};

__global__ __launch_bounds__(256) void dsa_build_rows_kernel(const RowsParams p) {
  __shared__ int scratch[8];
  const int tid = threadIdx.x;
  const int b = blockIdx.x / p.max_q_len;
  const int ti = blockIdx.x - b * p.max_q_len;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  if (ti >= qlen) return;
  const int t = q0 + ti;
  int n = p.seq_lens[b] - qlen + ti + 1;
  n = n < 0 ? 0 : n;
  const int32_t* idx = p.indices + (int64_t)t * p.i_st;
  int32_t* rows = p.rows + (int64_t)t * p.r_st;
  const int per = (p.k + 255) / 256;
  const int lo = tid * per;
  int hi = lo + per;
  hi = hi < p.k ? hi : p.k;
  int cnt = 0;
  for (int i = lo; i < hi; i++) { const int v = idx[i]; cnt += v >= 0 && v < n; }
  const int lane = tid & 63, w = tid >> 6;
  int s = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(s, o, 64);
    if (lane >= o) s += v;
  }
  if (lane == 63) scratch[w] = s;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += scratch[i];
  int o = base + s - cnt;
  for (int i = lo; i < hi; i++) {
    const int v = idx[i];
    if (v >= 0 && v < n) {
      int pg = v / p.page_size;
      const int off = v - pg * p.page_size;
      pg = pg < p.max_blocks ? pg : p.max_blocks - 1;
      int64_t blk = p.block_table[(int64_t)b * p.bt_stride + pg];
      blk = blk < 0 ? 0 : (blk >= p.num_pages ? p.num_pages - 1 : blk);
      rows[o++] = (int32_t)(blk * p.page_size + off);
    }
  }
  if (tid == 255) p.counts[t] = base + s;                  // inclusive total of the last thread
}

}  // namespace mlahip
using namespace mlahip;

extern "C" int dsa_topk(const float* logits, int64_t logits_stride, const int32_t* seq_lens, const int32_t* query_start_loc,
                        int32_t batch, int32_t max_q_len, int32_t k, int32_t* out_indices, int64_t out_stride,
                        hipStream_t stream) {
  MLA_REQUIRE(logits && seq_lens && out_indices, MLA_ERR_NULL, "dsa_topk: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && k >= 1 && out_stride >= k, MLA_ERR_SHAPE,
              "dsa_topk: batch=%d max_q_len=%d k=%d out_stride=%lld", batch, max_q_len, k, (long long)out_stride);
  MLA_REQUIRE(logits_stride < (1ll << 22), MLA_ERR_SHAPE, "dsa_topk: at most 2^22 keys per row");
  if (batch == 0) return MLA_OK;
  TopkParams p{logits, logits_stride, seq_lens, query_start_loc, batch, max_q_len, k, out_indices, out_stride};
  hipLaunchKernelGGL(dsa_topk_kernel, dim3(batch * max_q_len), dim3(kTopkThreads), 0, stream, p);
  return check_launch("dsa_topk_kernel");
}

extern "C" int dsa_build_rows(const int32_t* indices, int64_t indices_stride, const int32_t* block_table, int64_t bt_stride,
                              int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                              int32_t max_q_len, int32_t k, int32_t page_size, int64_t num_pages, int32_t* rows,
                              int64_t rows_stride, int32_t* counts, hipStream_t stream) {
  MLA_REQUIRE(indices && block_table && seq_lens && rows && counts, MLA_ERR_NULL, "dsa_build_rows: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && k >= 1 && page_size >= 1 && num_pages >= 1 && max_blocks >= 1 &&
                  rows_stride >= k && indices_stride >= k && num_pages * page_size < (1ll << 31),
              MLA_ERR_SHAPE, "dsa_build_rows: batch=%d max_q_len=%d k=%d page_size=%d", batch, max_q_len, k, page_size);
  if (batch == 0) return MLA_OK;
  RowsParams p{indices, indices_stride, block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len,
               k, page_size, num_pages, rows, rows_stride, counts};
  hipLaunchKernelGGL(dsa_build_rows_kernel, dim3(batch * max_q_len), dim3(256), 0, stream, p);
  return check_launch("dsa_build_rows_kernel");
}
