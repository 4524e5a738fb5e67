// DSA lightning indexer: fp8 score GEMM + weighted ReLU reduction over index heads.
//
// Replaces the score half of torch.ops.custom.npu_lightning_indexer as the reference calls it
// (src/omni_npu/v1/layers/attention/npu_dsa.py:92-103,
//  src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:133-144):
//   logit[t, s] = k_scale[s] * sum_h w[t,h] * relu(q8[t,h,:] . k8[s,:]),   s < visible(t)
// q8 / k8 are float8_e4m3fn (OCP), 128 wide; w already carries the per-(token, head) q scale unless a
// separate q_scale is passed.  The selection half is dsa_topk (topk.hip).
//
// Pure streaming kernel: a wavefront walks blocks of 32 keys (its equal share of all blocks of the launch).  A block
// (32 rows of 128 bytes and their 32 scales) travels global -> LDS in five copy instructions that bypass the registers,
// every one covering whole 128-byte lines (a lane that loaded its own row's bytes would touch 32 lines per instruction,
// each of them four times over), into a ring of four slots that belongs to the wavefront alone: no barrier anywhere.
// Lane (key = l % 32, half = l / 32) then reads bytes [64*half, 64*half + 64) of its key row from the slot and uses them
// as the B operand of 8 MFMA 32x32x16 fp8 steps per head block (the k order inside a step is free as long as A
// uses the same one).  A = the query's 64 heads x 128, held in 32 registers.  In the accumulator layout
// a lane owns one key and 16 of the 32 heads of a block, so the weighted ReLU sum is 32 in-lane FMAs plus
// one exchange between the two half-waves.
#include "mla_common.hpp"

namespace mlahip {

constexpr int kIdxDim = 128;
constexpr int kIdxRing = 4;                           // ring slots per wavefront (3 blocks requested ahead)
constexpr int kIdxSlotB = 32 * kIdxDim + 32 * 4;      // 4224: 32 key rows + their 32 scales
constexpr int kIdxLdsB = 4 * kIdxRing * kIdxSlotB;    // 67584 per workgroup of four wavefronts, two workgroups per CU
constexpr int kIdxCopies = 5;                         // copy instructions per block

struct IndexerParams {
  const uint8_t* q8; int64_t q_st, q_sh;              // bytes
  const float* weights; int64_t w_st;                 // [T, H]
  const float* q_scale; int64_t qs_st;                // optional [T, H]
  const uint8_t* k8; int64_t k_sp, k_sr;              // bytes: page stride, row stride
  const float* k_scale; int64_t ks_sp;                // elements: page stride (row stride 1)
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, num_heads, page_size;
  int64_t num_pages;
  float* logits; int64_t l_st;                        // [T, l_st]
};

__device__ __forceinline__ int idx_wave_sum(int v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}
__device__ __forceinline__ int idx_wave_max(int v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = max(v, __shfl_xor(v, d, 64));
  return v;
}

// The 32-key blocks of all query tokens, laid end to end, are dealt out to the wavefronts of the launch in equal
// contiguous shares (to within one block), whatever the individual context lengths; a share that crosses a token
// boundary is processed as two (or more) segments.  Every wavefront derives its share from the sequence lengths by
// itself (two passes: total, scan); there is no barrier in this kernel and no LDS is shared, so wavefronts are independent.
__global__ __launch_bounds__(256, 2) void dsa_indexer_fp8_kernel(const IndexerParams p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int key_l = lane & 31, half = lane >> 5;
  const int slots = p.batch * p.max_q_len;
  // visible keys of token slot s = (request, token inside the request); 0 for slots past a request's length
  auto limit_of = [&](int s) -> int {
    const int bb = s / p.max_q_len, tt = s - bb * p.max_q_len;
    const int ql0 = p.qsl ? p.qsl[bb + 1] - p.qsl[bb] : p.max_q_len;
    const int ql = ql0 < p.max_q_len ? ql0 : p.max_q_len;
    if (tt >= ql) return 0;
    const int lim = p.seq_lens[bb] - ql + tt + 1;
    return lim < 0 ? 0 : lim;
  };
  int seg_s, seg_off, remaining;
  {
    int tot = 0;
    for (int i = lane; i < slots; i += 64) tot += (limit_of(i) + 31) >> 5;
    tot = __builtin_amdgcn_readfirstlane(idx_wave_sum(tot));
    const int64_t nw = (int64_t)gridDim.x * 4, me = (int64_t)blockIdx.x * 4 + wave;
    const int64_t ub = me * tot / nw, ue = (me + 1) * tot / nw;
    if (ub == ue) return;
    int carry = 0, s0 = 0, pb0 = 0;
    for (int base = 0; base < slots; base += 64) {
      const int i = base + lane;
      const int c = i < slots ? (limit_of(i) + 31) >> 5 : 0;
      int pe = c;                                         // inclusive scan
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) { const int v = __shfl_up(pe, d, 64); pe += lane >= d ? v : 0; }
      pe += carry;
      const bool le = i < slots && pe <= ub;              // slot i ends at or before my first block
      s0 += __builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
      pb0 = max(pb0, idx_wave_max(le ? pe : 0));
      carry = __builtin_amdgcn_readlane(pe, 63);
    }
    seg_s = __builtin_amdgcn_readfirstlane(s0) - 1;
    seg_off = (int)ub - __builtin_amdgcn_readfirstlane(pb0);
    remaining = (int)(ue - ub);
  }

  while (remaining > 0) {
  seg_s++;
  if (seg_s >= slots) break;
  const int b = seg_s / p.max_q_len;
  const int ti = seg_s - b * p.max_q_len;              // query token inside the request
  const int limit = limit_of(seg_s);                   // visible keys (right-down causal)
  const int blk_begin = seg_off;
  seg_off = 0;
  int take = ((limit + 31) >> 5) - blk_begin;
  take = take < remaining ? take : remaining;
  if (take <= 0) continue;
  remaining -= take;
  const int t = (p.qsl ? p.qsl[b] : b * p.max_q_len) + ti;
  const int key_begin = blk_begin * 32;
  int key_end = key_begin + take * 32;
  key_end = key_end < limit ? key_end : limit;

  // A operand: head = hb*32 + key_l (as row index), bytes [64*half, +64) of that head's query row
  long qa[2][8];
  float wr[2][16];
#pragma unroll
  for (int hb = 0; hb < 2; hb++) {
    const uint8_t* qrow = p.q8 + (int64_t)t * p.q_st + (int64_t)(hb * 32 + key_l) * p.q_sh + half * 64;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      u32x4 v = *(const u32x4*)(qrow + j * 16);
      qa[hb][2 * j] = (long)(((uint64_t)v[1] << 32) | v[0]);
      qa[hb][2 * j + 1] = (long)(((uint64_t)v[3] << 32) | v[2]);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) wr[hb][r] = p.weights[(int64_t)t * p.w_st + hb * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
  }
  if (p.q_scale) {                                      // (all 32 scales asked for together, not one round trip each)
    float qs[2][16];
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int r = 0; r < 16; r++) qs[hb][r] = p.q_scale[(int64_t)t * p.qs_st + hb * 32 + 8 * (r >> 2) + 4 * half + (r & 3)];
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int r = 0; r < 16; r++) wr[hb][r] *= qs[hb][r];
  }

  // Key blocks are requested kIdxRing - 1 blocks ahead of their use: a block is 4 KiB per wavefront, and only what is in
  // flight hides the memory latency.  Pages hold a whole number of 32-key blocks (checked on the host), so the page
  // number of a block is a scalar (one scalar load of the block table) and the block's rows are contiguous in the page.
  // Slot layout: row r at r * 128, its 16-byte granule g at position g ^ ((r >> 1) & 7), so that the sixteen lanes of a
  // read phase (rows of both parities, one logical granule) hit sixteen different bank groups; the scales behind the rows.
  // Rows of the last block past the visible keys are read too (they lie inside the page) and never used.
  const uint32_t ring = lds_addr_of(lds) + (uint32_t)wave * (kIdxRing * kIdxSlotB);
  const char* ring_p = lds + wave * (kIdxRing * kIdxSlotB);
  uint32_t src_off[4];                                  // copy i, lane l: row 8 i + l / 8, granule (l % 8) ^ swizzle(row)
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = i * 8 + (lane >> 3);
    src_off[i] = (uint32_t)(r * (int)p.k_sr + 16 * ((lane & 7) ^ ((r >> 1) & 7)));
  }
  int nxt_pg = key_begin / p.page_size;                 // page and row offset of the next block to request
  int nxt_off = key_begin - nxt_pg * p.page_size;
  auto issue_block = [&](int slot) {
    const int pgc = nxt_pg < p.max_blocks ? nxt_pg : p.max_blocks - 1;
    int64_t blk = ((const __attribute__((address_space(4))) int32_t*)p.block_table)[(int64_t)b * p.bt_stride + pgc];
    blk = blk < 0 ? 0 : (blk >= p.num_pages ? p.num_pages - 1 : blk);
    const uint8_t* rows = p.k8 + blk * p.k_sp + (int64_t)nxt_off * p.k_sr;
    const float* sc = p.k_scale + blk * p.ks_sp + nxt_off;
    const uint32_t dst = ring + (uint32_t)slot * kIdxSlotB;
#pragma unroll
    for (int i = 0; i < 4; i++) dma16_sv_nt(rows, src_off[i], dst + i * 1024);
    dma4_sv_lo32(sc, (uint32_t)lane * 4, dst + 32 * kIdxDim);
    nxt_off += 32;
    if (nxt_off >= p.page_size) { nxt_off = 0; nxt_pg++; }
  };
  const int nblk = (key_end - key_begin + 31) >> 5;
#pragma unroll
  for (int i = 0; i < kIdxRing - 1; i++)
    if (i < nblk) issue_block(i);
  const int rd_row = key_l * kIdxDim, rd_swz = (key_l >> 1) & 7;
  for (int g = 0; g < nblk; g++) {
    const int slot = g & (kIdxRing - 1);
    if (g + kIdxRing - 1 < nblk) issue_block((g + kIdxRing - 1) & (kIdxRing - 1));
    // this block has landed when at most the copies of the younger blocks are outstanding (the logits stores in between
    // count too: at worst the wait is a little longer than needed)
    const int younger = nblk - 1 - g;
    if (younger >= 3) MLA_WAIT_VMCNT(15);
    else if (younger == 2) MLA_WAIT_VMCNT(10);
    else if (younger == 1) MLA_WAIT_VMCNT(5);
    else MLA_WAIT_VMCNT(0);
    const char* sp = ring_p + slot * kIdxSlotB;
    u32x4 kb[4];
#pragma unroll
    for (int j = 0; j < 4; j++) kb[j] = *(const u32x4*)(sp + rd_row + (((4 * half + j) ^ rd_swz) << 4));
    const float ks = *(const float*)(sp + 32 * kIdxDim + key_l * 4);
    f32x16 c0, c1;
#pragma unroll
    for (int r = 0; r < 16; r++) { c0[r] = 0.f; c1[r] = 0.f; }
#pragma unroll
    for (int kk = 0; kk < 8; kk++) {
      const u32x4 v = kb[kk >> 1];
      const long bop = (kk & 1) ? (long)(((uint64_t)v[3] << 32) | v[2]) : (long)(((uint64_t)v[1] << 32) | v[0]);
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(qa[0][kk], bop, c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(qa[1][kk], bop, c1, 0, 0, 0);
    }
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      acc = fmaf(wr[0][r], fmaxf(c0[r], 0.f), acc);
      acc = fmaf(wr[1][r], fmaxf(c1[r], 0.f), acc);
    }
    acc += xor32(acc);
    const int key = key_begin + 32 * g + key_l;
    if (half == 0) p.logits[(int64_t)t * p.l_st + key] = key < limit ? acc * ks : -INFINITY;
  }
  }  // segments
}

// Per-row e4m3 quantisation of 128-wide bf16 rows (one fp32 scale = amax/448 per row, 1.0 for an all-zero row),
// optionally scattered through a slot mapping into a paged fp8 cache + scale cache: the indexer-K write of
// src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:116-121 with quantisation fused in, and
// the query quantisation (no slot mapping).  One wavefront per row, lane l owns elements 2l, 2l+1.
struct QuantRows {
  const __bf16* src; int64_t src_stride, rows;
  const int64_t* slots;
  uint8_t* dst8; int64_t d_sp, d_sr;
  float* dscale; int64_t s_sp;
  int32_t page_size; int64_t num_pages;
};

__device__ __forceinline__ void quant_row(const __bf16* src, int64_t src_stride, int64_t rows, const int64_t* slots,
                                          uint8_t* dst8, int64_t d_sp, int64_t d_sr, float* dscale, int64_t s_sp,
                                          int32_t page_size, int64_t num_pages, int64_t r) {
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  int64_t slot = slots ? slots[r] : r;
  if (slot < 0 || slot >= num_pages * page_size) return;
  const int64_t pg = slot / page_size, off = slot - pg * page_size;
  const bf16x2 v = *(const bf16x2*)(src + r * src_stride + lane * 2);
  const float x0 = (float)v[0], x1 = (float)v[1];
  float amax = fmaxf(fabsf(x0), fabsf(x1));
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
  const float scale = amax > 0.f ? amax / 448.f : 1.f;
  const float y0 = fminf(fmaxf(x0 / scale, -448.f), 448.f), y1 = fminf(fmaxf(x1 / scale, -448.f), 448.f);
  const int w = __builtin_amdgcn_cvt_pk_fp8_f32(y0, y1, 0, false);
  *(uint16_t*)(dst8 + pg * d_sp + off * d_sr + lane * 2) = (uint16_t)(w & 0xFFFF);
  if (lane == 0) dscale[pg * s_sp + off] = scale;
}

__global__ __launch_bounds__(256) void dsa_quant_rows_kernel(const __bf16* src, int64_t src_stride, int64_t rows,
                                                             const int64_t* slots, uint8_t* dst8, int64_t d_sp, int64_t d_sr,
                                                             float* dscale, int64_t s_sp, int32_t page_size,
                                                             int64_t num_pages) {
  quant_row(src, src_stride, rows, slots, dst8, d_sp, d_sr, dscale, s_sp, page_size, num_pages,
            (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6));
}

// Two row sets in one launch (the indexer's step: the query rows into plain buffers, the new key rows into the cache):
// the first a_blocks workgroups take set a, the others set b.
__global__ __launch_bounds__(256) void dsa_quant_rows2_kernel(const QuantRows a, const QuantRows b, int32_t a_blocks) {
  const bool first = (int)blockIdx.x < a_blocks;
  const QuantRows& q = first ? a : b;
  quant_row(q.src, q.src_stride, q.rows, q.slots, q.dst8, q.d_sp, q.d_sr, q.dscale, q.s_sp, q.page_size, q.num_pages,
            (int64_t)(first ? blockIdx.x : blockIdx.x - a_blocks) * 4 + (threadIdx.x >> 6));
}

}  // namespace mlahip
using namespace mlahip;

// dsa_quant_rows_fp8 of the query rows (plain outputs) and of the new key rows (into the paged index-key cache) in one launch.
extern "C" int dsa_quant_qk_fp8(const void* q, int64_t q_stride, int64_t q_rows, void* q8, float* q_scale, const void* k,
                                int64_t k_stride, int64_t k_rows, const int64_t* slot_mapping, void* k8_cache,
                                int64_t cache_page_stride_bytes, int64_t cache_row_stride_bytes, float* scale_cache,
                                int64_t scale_page_stride, int32_t page_size, int64_t num_pages, hipStream_t stream) {
  MLA_REQUIRE(q && q8 && q_scale && k && slot_mapping && k8_cache && scale_cache, MLA_ERR_NULL,
              "dsa_quant_qk_fp8: null pointer argument");
  MLA_REQUIRE(q_rows >= 0 && k_rows >= 0 && page_size >= 1 && num_pages >= 1 && q_stride % 2 == 0 && k_stride % 2 == 0 &&
                  cache_row_stride_bytes >= 128 && cache_row_stride_bytes % 2 == 0 && cache_page_stride_bytes % 2 == 0 &&
                  (uintptr_t)q % 4 == 0 && (uintptr_t)k % 4 == 0 && (uintptr_t)q8 % 2 == 0 && (uintptr_t)k8_cache % 2 == 0 &&
                  q_rows < (1ll << 31) && k_rows < (1ll << 31),
              MLA_ERR_SHAPE, "dsa_quant_qk_fp8: q_rows=%lld k_rows=%lld page_size=%d", (long long)q_rows, (long long)k_rows,
              page_size);
  if (q_rows + k_rows == 0) return MLA_OK;
  // (set a has no slot mapping: row r is "slot" r of one page that holds them all)
  const QuantRows a{(const __bf16*)q, q_stride, q_rows, nullptr, (uint8_t*)q8, 0, 128, q_scale, 0,
                    (int32_t)(q_rows > 0 ? q_rows : 1), 1};
  const QuantRows b{(const __bf16*)k, k_stride, k_rows, slot_mapping, (uint8_t*)k8_cache, cache_page_stride_bytes,
                    cache_row_stride_bytes, scale_cache, scale_page_stride, page_size, num_pages};
  const int64_t a_blocks = (q_rows + 3) / 4, b_blocks = (k_rows + 3) / 4;
  hipLaunchKernelGGL(dsa_quant_rows2_kernel, dim3((unsigned)(a_blocks + b_blocks)), dim3(256), 0, stream, a, b,
                     (int32_t)a_blocks);
  return check_launch("dsa_quant_rows2_kernel");
}

extern "C" int dsa_quant_rows_fp8(const void* src, int64_t src_stride, int64_t rows, const int64_t* slot_mapping,
                                  void* dst8, int64_t dst_page_stride_bytes, int64_t dst_row_stride_bytes,
                                  float* dst_scale, int64_t scale_page_stride, int32_t page_size, int64_t num_pages,
                                  hipStream_t stream) {
  MLA_REQUIRE(src && dst8 && dst_scale, MLA_ERR_NULL, "dsa_quant_rows_fp8: null pointer argument");
  MLA_REQUIRE(rows >= 0 && page_size >= 1 && num_pages >= 1 && src_stride % 2 == 0 && dst_row_stride_bytes >= 128 &&
                  (uintptr_t)src % 4 == 0 && (uintptr_t)dst8 % 2 == 0 && dst_row_stride_bytes % 2 == 0 &&
                  dst_page_stride_bytes % 2 == 0,
              MLA_ERR_SHAPE, "dsa_quant_rows_fp8: rows=%lld page_size=%d", (long long)rows, page_size);
  if (rows == 0) return MLA_OK;
  hipLaunchKernelGGL(dsa_quant_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream, (const __bf16*)src,
                     src_stride, rows, slot_mapping, (uint8_t*)dst8, dst_page_stride_bytes, dst_row_stride_bytes, dst_scale,
                     scale_page_stride, page_size, num_pages);
  return check_launch("dsa_quant_rows_kernel");
}

extern "C" int dsa_indexer_scores_fp8(const void* q8, int64_t q_stride_t, int64_t q_stride_h, const float* weights,
                                      int64_t w_stride_t, const float* q_scale, int64_t qs_stride_t, const void* k8_cache,
                                      int64_t k_page_stride, int64_t k_row_stride, const float* k_scale_cache,
                                      int64_t ks_page_stride, int64_t num_pages, int32_t page_size,
                                      const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                      const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                      int32_t max_q_len, int32_t num_heads, int32_t max_seq_len, float* logits,
                                      int64_t logits_stride, hipStream_t stream) {
  MLA_REQUIRE(q8 && weights && k8_cache && k_scale_cache && block_table && seq_lens && logits, MLA_ERR_NULL,
              "dsa_indexer_scores_fp8: null pointer argument");
  MLA_REQUIRE(num_heads == 64, MLA_ERR_UNSUPPORTED, "dsa_indexer_scores_fp8: 64 index heads only (got %d)", num_heads);
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && page_size >= 32 && page_size % 32 == 0 && num_pages >= 1 && max_blocks >= 1 &&
                  max_seq_len >= 1,
              MLA_ERR_SHAPE, "dsa_indexer_scores_fp8: batch=%d max_q_len=%d page_size=%d max_seq_len=%d", batch, max_q_len,
              page_size, max_seq_len);
  MLA_REQUIRE(k_row_stride >= kIdxDim && k_row_stride <= (1 << 20), MLA_ERR_SHAPE,
              "dsa_indexer_scores_fp8: key row stride %lld bytes", (long long)k_row_stride);
  MLA_REQUIRE(q_stride_t % 16 == 0 && q_stride_h % 16 == 0 && k_page_stride % 16 == 0 && k_row_stride % 16 == 0 &&
                  (uintptr_t)q8 % 16 == 0 && (uintptr_t)k8_cache % 16 == 0,
              MLA_ERR_SHAPE, "dsa_indexer_scores_fp8: fp8 rows must be 16-byte aligned");
  MLA_REQUIRE(logits_stride >= (int64_t)((max_seq_len + 31) / 32) * 32, MLA_ERR_SHAPE,
              "dsa_indexer_scores_fp8: logits rows must hold max_seq_len rounded up to 32 (%lld < %d)",
              (long long)logits_stride, ((max_seq_len + 31) / 32) * 32);
  if (batch == 0) return MLA_OK;
  MLA_REQUIRE((int64_t)batch * max_q_len <= 65535, MLA_ERR_SHAPE, "dsa_indexer_scores_fp8: too many query tokens");
  IndexerParams p;
  p.q8 = (const uint8_t*)q8; p.q_st = q_stride_t; p.q_sh = q_stride_h;
  p.weights = weights; p.w_st = w_stride_t; p.q_scale = q_scale; p.qs_st = qs_stride_t;
  p.k8 = (const uint8_t*)k8_cache; p.k_sp = k_page_stride; p.k_sr = k_row_stride;
  p.k_scale = k_scale_cache; p.ks_sp = ks_page_stride;
  p.block_table = block_table; p.bt_stride = bt_stride; p.max_blocks = max_blocks;
  p.seq_lens = seq_lens; p.qsl = query_start_loc;
  p.batch = batch; p.max_q_len = max_q_len; p.num_heads = num_heads; p.page_size = page_size; p.num_pages = num_pages;
  p.logits = logits; p.l_st = logits_stride;
  // two workgroups per compute unit (what their LDS rings allow), never more wavefronts than 32-key blocks
  static int num_cus = 0;
  if (num_cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&num_cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        num_cus <= 0)
      num_cus = 256;
  }
  const int64_t max_blocks_total = (int64_t)batch * max_q_len * ((max_seq_len + 31) / 32);
  int64_t wgs = 2 * (int64_t)num_cus;
  if (wgs * 4 > max_blocks_total) wgs = (max_blocks_total + 3) / 4;
  if (wgs < 1) wgs = 1;
  const int rc = ensure_dynamic_lds((const void*)dsa_indexer_fp8_kernel, kIdxLdsB, "dsa_indexer_scores_fp8");
  if (rc != MLA_OK) return rc;
  hipLaunchKernelGGL(dsa_indexer_fp8_kernel, dim3((unsigned)wgs), dim3(256), kIdxLdsB, stream, p);
  return check_launch("dsa_indexer_fp8_kernel");
}
