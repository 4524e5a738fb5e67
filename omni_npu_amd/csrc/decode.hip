// Absorbed-MLA paged decode for gfx950 (bf16 cache), split-KV, plus the split reduction.
//
// Replaces the reference's decode call of npu_fused_infer_attention_score
// (src/omni_npu/attention/backends/mla.py:781-804): for sequence b, head n, query token t
//   s_j = scale * (ql[t,n] . Kc[j] + qr[t,n] . Kr[j]),  j < L_b - (q_len-1-t)   (right-down causal)
//   o   = sum_j softmax(s)_j * Kc[j]
// with ONE latent KV row (512 + 64) shared by all heads.
//
// Work decomposition.  One workgroup = 4 wavefronts = (sequence b, KV split s, group of 128 query
// rows), a query row being a (query token, head) pair.  Each wavefront owns 32 rows and keeps, in
// registers, their whole 576-wide query (as the B operand of S^T = K . Q^T, 36 k-steps) and their
// 512 x 32 fp32 output accumulator O^T (16 MFMA 32x32 blocks).  K tiles of 64 tokens are copied
// global -> LDS without touching registers, double buffered, the nope part (64 x 1024 B) and the rope
// part (64 x 128 B) as two swizzled regions.  Per 32 tokens a wavefront issues 36 MFMA 32x32x16 for
// S^T = K Q^T (A operand = K rows, 16-byte LDS reads), an online-softmax update, and 32 MFMA for
// O^T += V^T P^T, whose A operand V^T (V = first 512 columns of the same K rows) comes from
// transposed LDS reads.  Computing the transposed products makes the accumulator layout of S^T the
// B-operand layout of P^T, so P never leaves registers.
//
// Each workgroup writes a normalised fp32 partial and its log-sum-exp; mla_splitkv_reduce_kernel folds the
// splits with the N-way merge of src/omni_npu/attention/ops.py:109-141 and writes bf16.
#include <cstdlib>
#include "mla_common.hpp"
#include "decode_v2_params.hpp"

namespace mlahip {

constexpr int kTile = 64;                          // tokens per LDS tile
constexpr int kNopeRowB = kDNope * 2;              // 1024
constexpr int kRopeRowB = kDRope * 2;              // 128
constexpr int kNopeTileB = kTile * kNopeRowB;      // 65536
constexpr int kRopeTileB = kTile * kRopeRowB;      // 8192
constexpr int kBufB = kNopeTileB + kRopeTileB;     // 73728
constexpr int kDecodeLdsB = 2 * kBufB;             // 147456
constexpr int kRowsPerWg = 128;
// KV source of the kernel: paged bf16 cache, per-token row list over a bf16 cache, paged fp8 block-scaled cache
constexpr int kModeDense = 0, kModeSparse = 1, kModeFp8 = 2;
// fp8 mode: one bf16 tile buffer (dequantised) + two raw staging buffers of 44 KiB (64 rows x 656 B, rounded up)
constexpr int kFp8RowB = 656, kFp8ScaleOff = 512, kFp8RopeOff = 528;
constexpr int kRawStageB = 44 * 1024;
constexpr int kFp8LdsB = kBufB + 2 * kRawStageB;      // 163840 = all of the LDS
#ifndef MLA_QK_AHEAD
#define MLA_QK_AHEAD 2
#endif
#ifndef MLA_PV_AHEAD
#define MLA_PV_AHEAD 2
#endif
constexpr int kQkAhead = MLA_QK_AHEAD;               // LDS read-ahead depth, in MFMA steps
constexpr int kPvAhead = MLA_PV_AHEAD;

// 16-byte granule swizzles (functions of row % 16).  A nope row has 64 granules, a rope row 8.
// They spread (i) 16 consecutive rows at one column over 16 distinct 16-byte bank groups for the
// row-wise reads and (ii) 4 consecutive rows x 64 bytes over distinct bank groups for the transposed
// reads.
__device__ __forceinline__ int swz_nope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r1 ^ r3) << 3) | (r0 << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int swz_rope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r0 ^ r3) << 2) | (r1 << 1) | r2;
}

struct DecodeParams {
  const __bf16* q_nope; int64_t qn_st, qn_sh;
  const __bf16* q_rope; int64_t qr_st, qr_sh;
  const __bf16* nope; int64_t nope_sp, nope_sr;
  const __bf16* rope; int64_t rope_sp, rope_sr;
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks;
  const int32_t* seq_lens;
  const int32_t* qsl;            // [B+1] or null
  int32_t batch, max_q_len, num_heads;
  int64_t num_pages;
  float scale_log2;              // scale * log2(e)
  _Float16* o_part;              // [B*S, R_max, 512] fp16, normalised
  float* lse_part;               // [B*S, R_max]   (natural log)
  int32_t num_splits;
  // sparse variant: the keys of "sequence" b are the flat cache rows sparse_rows[b, 0 .. seq_lens[b])
  const int32_t* sparse_rows; int64_t sparse_stride; int32_t page_size;
};

// Issue the global -> LDS copies of one 64-token tile (18 x 16 B per lane).  Row bases are
// wave-uniform (scalar registers).  Wave w copies the nope rows r with r % 16 in [4w, 4w+4), so that
// only four distinct per-lane granule permutations (dma_off, bytes) are needed.
template <int kMode>
__device__ __forceinline__ void issue_tile(const DecodeParams& p, int b, int tile, int L, uint32_t buf, int wave, int lane,
                                           const uint32_t (&dma_off)[4], const uint32_t (&rope_off)[2]) {
  const int tok0 = tile * kTile;
  const int last = L - 1 - tok0;                   // last valid row of this tile (>= 0)
  constexpr bool kSparse = kMode == kModeSparse;
  if constexpr (kSparse) {
    // every row has its own flat cache row id, read through the scalar cache
    const __attribute__((address_space(4))) int32_t* rows =
        (const __attribute__((address_space(4))) int32_t*)(p.sparse_rows + (int64_t)b * p.sparse_stride + tok0);
    const int64_t max_row = p.num_pages * p.page_size - 1;
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const int r = q * 16 + wave * 4 + j;
        const int re = r < last ? r : last;
        int64_t slot = rows[re];
        slot = slot < 0 ? 0 : (slot > max_row ? max_row : slot);
        const char* rowp = (const char*)(p.nope + slot * p.nope_sr);     // pages are contiguous (checked on the host)
        dma16_sv(rowp, dma_off[j], buf + r * kNopeRowB);
      }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int r0 = wave * 16 + j * 8;
      const int r = r0 + (lane >> 3);
      const int re = r < last ? r : last;
      int64_t slot = p.sparse_rows[(int64_t)b * p.sparse_stride + tok0 + re];
      slot = slot < 0 ? 0 : (slot > max_row ? max_row : slot);
      const char* g = (const char*)(p.rope + slot * p.rope_sr) + rope_off[j];
      dma16_v(g, buf + kNopeTileB + r0 * kRopeRowB);
    }
    return;
  }
  int page = tok0 / kPage;
  page = page < p.max_blocks ? page : p.max_blocks - 1;
  int64_t blk = __builtin_amdgcn_readfirstlane(p.block_table[(int64_t)b * p.bt_stride + page]);
  blk = blk < 0 ? 0 : (blk >= p.num_pages ? p.num_pages - 1 : blk);
  const int row_in_page0 = tok0 % kPage;
  const char* nope_pg = (const char*)(p.nope + blk * p.nope_sp) + (int64_t)row_in_page0 * p.nope_sr * 2;
  const char* rope_pg = (const char*)(p.rope + blk * p.rope_sp) + (int64_t)row_in_page0 * p.rope_sr * 2;
#pragma unroll
  for (int q = 0; q < 4; q++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int r = q * 16 + wave * 4 + j;
      const int re = r < last ? r : last;          // rows past the end re-read the last valid row
      const char* rowp = nope_pg + (int64_t)re * p.nope_sr * 2;
      dma16_sv(rowp, dma_off[j], buf + r * kNopeRowB);
    }
  // rope: 8 lanes per row, wave w copies rows 16w .. 16w+15 in two steps of 8 rows
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int r0 = wave * 16 + j * 8;              // first row of this step (uniform)
    const int r = r0 + (lane >> 3);
    const int re = r < last ? r : last;
    const char* g = rope_pg + (int64_t)re * p.rope_sr * 2 + rope_off[j];
    dma16_v(g, buf + kNopeTileB + r0 * kRopeRowB);
  }
}

// fp8 mode: a 64-token tile is 64 x 656 contiguous bytes inside its page; copy it linearly (44 wave copies of
// 1 KiB, 11 per wave; the tail copies re-read the last granule of the tile).
__device__ __forceinline__ void issue_raw_tile(const DecodeParams& p, int b, int tile, uint32_t stage, int wave, int lane) {
  const int tok0 = tile * kTile;
  int page = tok0 / kPage;
  page = page < p.max_blocks ? page : p.max_blocks - 1;
  int64_t blk = __builtin_amdgcn_readfirstlane(p.block_table[(int64_t)b * p.bt_stride + page]);
  blk = blk < 0 ? 0 : (blk >= p.num_pages ? p.num_pages - 1 : blk);
  const char* src = (const char*)p.nope + blk * p.nope_sp + (int64_t)(tok0 % kPage) * kFp8RowB;   // strides in bytes here
  constexpr int kGranules = kTile * kFp8RowB / 16;   // 2624
#pragma unroll
  for (int i = 0; i < 11; i++) {
    const int wi = i * 4 + wave;
    int g = wi * 64 + lane;
    g = g < kGranules ? g : kGranules - 1;
    dma16_sv(src, (uint32_t)g << 4, stage + wi * 1024);
  }
}

// Dequantise the raw tile into the swizzled bf16 tile the MFMA phases read: x = e4m3 * block scale, rounded to
// bf16; rows past `valid` become zeros (their cache bytes are not defined).
__device__ __forceinline__ void dequant_tile(const char* raw, char* tile, int valid, int tid) {
#pragma unroll 2
  for (int it = 0; it < 8; it++) {
    const int u = it * 256 + tid;
    const int r = u >> 5, c = u & 31;                 // row, 16-element chunk
    const u32x4 w = *(const u32x4*)(raw + r * kFp8RowB + c * 16);
    const float sc = r < valid ? *(const float*)(raw + r * kFp8RowB + kFp8ScaleOff + (c >> 3) * 4) : 0.f;
    u32x4 lo, hi;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], false);
      const f32x2 bq = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], true);
      bf16x2 x, y;
      x[0] = (__bf16)(r < valid ? a[0] * sc : 0.f); x[1] = (__bf16)(r < valid ? a[1] * sc : 0.f);
      y[0] = (__bf16)(r < valid ? bq[0] * sc : 0.f); y[1] = (__bf16)(r < valid ? bq[1] * sc : 0.f);
      const uint32_t px = __builtin_bit_cast(uint32_t, x), py = __builtin_bit_cast(uint32_t, y);
      if (j < 2) { lo[2 * j] = px; lo[2 * j + 1] = py; } else { hi[2 * (j - 2)] = px; hi[2 * (j - 2) + 1] = py; }
    }
    const int f = swz_nope(r & 15);
    *(u32x4*)(tile + r * kNopeRowB + (((2 * c) ^ f) << 4)) = lo;
    *(u32x4*)(tile + r * kNopeRowB + (((2 * c + 1) ^ f) << 4)) = hi;
  }
#pragma unroll
  for (int it = 0; it < 2; it++) {
    const int u = it * 256 + tid;
    const int r = u >> 3, c = u & 7;
    u32x4 w = *(const u32x4*)(raw + r * kFp8RowB + kFp8RopeOff + c * 16);
    if (r >= valid) w = u32x4{0, 0, 0, 0};
    *(u32x4*)(tile + kNopeTileB + r * kRopeRowB + ((c ^ swz_rope(r & 15)) << 4)) = w;
  }
}

template <int kMode>
__global__ __launch_bounds__(256, 1) void mla_decode_bf16_kernel(const DecodeParams p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h32 = lane & 31;
  const int half = lane >> 5;
  const int split = blockIdx.x;
  const int b = blockIdx.y;
  const int grp = blockIdx.z;

  const int L = p.seq_lens[b];
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  qlen = qlen < p.max_q_len ? qlen : p.max_q_len;
  const int rows = qlen * p.num_heads;
  const int r_max = p.max_q_len * p.num_heads;
  if (grp * kRowsPerWg >= r_max) return;

  const int row = grp * kRowsPerWg + wave * 32 + h32;        // this lane's query row
  const bool row_ok = row < rows && L > 0;
  const int t_local = row / p.num_heads;
  const int head = row - t_local * p.num_heads;
  int limit = row_ok ? (L - qlen + t_local + 1) : 0;         // number of visible keys
  limit = limit < 0 ? 0 : limit;

  const int64_t part_row = ((int64_t)b * p.num_splits + split) * r_max + row;

  // ---- token range of this split (whole tiles) ----
  const int tiles_total = (L + kTile - 1) / kTile;
  const int tps = (tiles_total + p.num_splits - 1) / p.num_splits;
  const int tile_begin = split * tps;
  int tile_end = tile_begin + tps;
  tile_end = tile_end < tiles_total ? tile_end : tiles_total;

  if (tile_begin >= tile_end || grp * kRowsPerWg >= rows) {   // empty split / no rows: uniform per workgroup
    if (row < r_max && half == 0) p.lse_part[part_row] = -INFINITY;
    return;
  }

  // ---- prologue: first tile in flight, then the query into registers ----
  // per-lane source permutations of the copies (the LDS side is linear in the lane index)
  uint32_t dma_off[4];
#pragma unroll
  for (int j = 0; j < 4; j++) dma_off[j] = (uint32_t)((lane ^ swz_nope((wave * 4 + j) & 15)) << 4);
  uint32_t rope_off[2];          // rope step j copies rows 16*wave + 8j + lane/8, granule slot lane%8
#pragma unroll
  for (int j = 0; j < 2; j++) rope_off[j] = (uint32_t)(((lane & 7) ^ swz_rope(j * 8 + (lane >> 3))) << 4);
  const uint32_t lds0 = lds_addr_of(lds);
  if constexpr (kMode == kModeFp8) issue_raw_tile(p, b, tile_begin, lds0 + kBufB, wave, lane);
  else issue_tile<kMode>(p, b, tile_begin, L, lds0, wave, lane, dma_off, rope_off);

  bf16x8 qf[36];
  {
    // rows past the end read row 0 of the first token (valid memory) and are zeroed afterwards
    const int64_t tq = row_ok ? (q0 + t_local) : q0;
    const int64_t hq = row_ok ? head : 0;
    const __bf16* qn = p.q_nope + tq * p.qn_st + hq * p.qn_sh + half * 8;
    const __bf16* qr = p.q_rope + tq * p.qr_st + hq * p.qr_sh + half * 8;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int kk = 0; kk < 32; kk++) { bf16x8 v = *(const bf16x8*)(qn + kk * 16); qf[kk] = row_ok ? v : zero; }
#pragma unroll
    for (int kk = 0; kk < 4; kk++) { bf16x8 v = *(const bf16x8*)(qr + kk * 16); qf[32 + kk] = row_ok ? v : zero; }
  }

  f32x16 acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  float m_run = -INFINITY;    // running max (log2 domain), identical in both half-waves
  float l_run = 0.f;          // running sum of this lane's 16-token slices

  // ---- per-lane LDS offsets (the swizzle touches only the low 4 bits of a granule index, so a
  // handful of offsets plus compile-time immediates cover every read) ----
  const int fk = swz_nope(h32 & 15);
  const int fr = swz_rope(h32 & 15);
  int koff[8], roff[4];
#pragma unroll
  for (int j = 0; j < 8; j++) koff[j] = h32 * kNopeRowB + (((j * 2 + half) ^ fk) << 4);     // + (kk/8)*256 + tb*32768
#pragma unroll
  for (int j = 0; j < 4; j++) roff[j] = kNopeTileB + h32 * kRopeRowB + (((j * 2 + half) ^ fr) << 4);
  // transposed V reads: lane (g16 = lane/16, j = lane%16) points at token 4*(g16/2) + j/4 (+8*rd),
  // columns 16*(g16%2) + 4*(j%4) .. +3 of the 32-wide d block db; granule = db*4 + cl
  const int g16 = lane >> 4, j16 = lane & 15;
  const int v_row = 4 * (g16 >> 1) + (j16 >> 2);              // + 8*rd + 16*kb + 32*tb
  const int v_cl = 2 * (g16 & 1) + ((j16 & 3) >> 1);
  const int v_in = (j16 & 1) * 8;
  int voff[2][4];
#pragma unroll
  for (int rd = 0; rd < 2; rd++) {
    const int rr = v_row + 8 * rd;
    const int f = swz_nope(rr & 15);
#pragma unroll
    for (int dl = 0; dl < 4; dl++)                            // db = 4*dq + dl; + dq*256 + kb*16384 + tb*32768
      voff[rd][dl] = rr * kNopeRowB + v_in + ((((dl * 4 + v_cl) ^ f)) << 4);
  }

  for (int tile = tile_begin; tile < tile_end; tile++) {
    char* buf = lds;
    if constexpr (kMode == kModeFp8) {
      const int st = (tile - tile_begin) & 1;
      if (tile + 1 < tile_end) {
        issue_raw_tile(p, b, tile + 1, lds0 + kBufB + (st ^ 1) * kRawStageB, wave, lane);
        MLA_WAIT_VMCNT(11);
      } else {
        MLA_WAIT_VMCNT(0);
      }
      lds_barrier();                                          // raw tile landed for all four waves
      dequant_tile(lds + kBufB + st * kRawStageB, lds, L - tile * kTile, threadIdx.x);
      lds_barrier();                                          // bf16 tile complete
    } else {
      buf = lds + ((tile - tile_begin) & 1) * kBufB;
      if (tile + 1 < tile_end) {
        issue_tile<kMode>(p, b, tile + 1, L, lds0 + ((tile + 1 - tile_begin) & 1) * kBufB, wave, lane, dma_off, rope_off);
        MLA_WAIT_VMCNT(18);
      } else {
        MLA_WAIT_VMCNT(0);
      }
      lds_barrier();                                          // tile visible to all four waves
    }

    const int tok_base = tile * kTile;
#pragma unroll 1
    for (int tb = 0; tb < 2; tb++) {
      if (tok_base + tb * 32 >= L) break;                     // uniform: nothing visible in this block
      // ---- S^T = K Q^T : 32 tokens x 32 rows ----
      f32x16 s;
#pragma unroll
      for (int r = 0; r < 16; r++) s[r] = 0.f;
      // LDS reads run kQkAhead k-steps ahead of the MFMAs that consume them
      const char* kb_ptr = buf + tb * 32 * kNopeRowB;
      const char* rb_ptr = buf + tb * 32 * kRopeRowB;
      auto k_frag = [&](int kk) -> bf16x8 {
        return kk < 32 ? *(const bf16x8*)(kb_ptr + koff[kk & 7] + (kk >> 3) * 256)
                       : *(const bf16x8*)(rb_ptr + roff[kk & 3]);
      };
      bf16x8 ka[kQkAhead];
#pragma unroll
      for (int i = 0; i < kQkAhead; i++) ka[i] = k_frag(i);
#pragma unroll
      for (int kk = 0; kk < 36; kk++) {
        const bf16x8 a = ka[kk % kQkAhead];
        if (kk + kQkAhead < 36) ka[kk % kQkAhead] = k_frag(kk + kQkAhead);
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[kk], s, 0, 0, 0);
      }
      // ---- online softmax (log2 domain) ----
      const int tok_lane0 = tok_base + tb * 32 + 4 * half;
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int tok = tok_lane0 + 8 * (r >> 2) + (r & 3);
        s[r] = tok < limit ? s[r] * p.scale_log2 : -INFINITY;
        mx = fmaxf(mx, s[r]);
      }
      mx = fmaxf(mx, xor32(mx));
      const float m_new = fmaxf(m_run, mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = fast_exp2(m_run - m_safe);
      float psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        s[r] = fast_exp2(s[r] - m_safe);
        psum += s[r];
      }
      l_run = l_run * alpha + psum;
      m_run = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
        for (int i = 0; i < 16; i++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][r] *= alpha;
      }
      bf16x8 pb[2];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int e = 0; e < 8; e++) pb[kb][e] = (__bf16)s[kb * 8 + e];
      // ---- O^T += V^T P^T ----
      const char* vb = buf + tb * 32 * kNopeRowB;
      auto v_frag = [&](int st) -> bf16x8 {                    // step st = 2*db + kb
        const int db = st >> 1, kb = st & 1;
        bf16x4 lo = lds_read_tr16(vb + kb * 16 * kNopeRowB + voff[0][db & 3] + (db >> 2) * 256);
        bf16x4 hi = lds_read_tr16(vb + kb * 16 * kNopeRowB + voff[1][db & 3] + (db >> 2) * 256);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      };
      bf16x8 va[kPvAhead];
#pragma unroll
      for (int i = 0; i < kPvAhead; i++) va[i] = v_frag(i);
#pragma unroll
      for (int st = 0; st < 32; st++) {
        const bf16x8 a = va[st % kPvAhead];
        if (st + kPvAhead < 32) va[st % kPvAhead] = v_frag(st + kPvAhead);
        acc[st >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[st & 1], acc[st >> 1], 0, 0, 0);
      }
    }
    lds_barrier();                                            // everyone is done reading this buffer
  }

  // ---- epilogue: normalised partial + lse ----
  const float l_tot = l_run + xor32(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (row < r_max) {
    if (half == 0) p.lse_part[part_row] = l_tot > 0.f ? (m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
    _Float16* op = p.o_part + part_row * kDNope + 4 * half;
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int db = 0; db < 16; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        h4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (_Float16)(acc[db][rg * 4 + e] * inv);
        *(h4*)(op + db * 32 + rg * 8) = v;
      }
  }
}

// N-way merge over the splits (src/omni_npu/attention/ops.py:109-141): one wavefront per query row.
struct ReduceParams {
  const _Float16* o_part; const float* lse_part;
  const int32_t* qsl;
  int32_t batch, max_q_len, num_heads, num_splits;
  __bf16* out; int64_t out_st, out_sh;
  float* lse_out; int64_t lse_st;      // optional [T, N]
};

__global__ __launch_bounds__(256) void mla_splitkv_reduce_kernel(const ReduceParams p) {
  const int lane = threadIdx.x & 63;
  const int r_max = p.max_q_len * p.num_heads;
  const int64_t gr = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (gr >= (int64_t)p.batch * r_max) return;
  const int b = gr / r_max;
  const int row = gr - (int64_t)b * r_max;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  qlen = qlen < p.max_q_len ? qlen : p.max_q_len;
  if (row >= qlen * p.num_heads) return;
  const int t_local = row / p.num_heads;
  const int head = row - t_local * p.num_heads;

  const int64_t base = ((int64_t)b * p.num_splits) * r_max + row;
  float m = -INFINITY;
  for (int s = 0; s < p.num_splits; s++) {
    float l = p.lse_part[base + (int64_t)s * r_max];
    l = l == INFINITY ? -INFINITY : l;
    m = fmaxf(m, l);
  }
  float tot = 0.f;
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (m != -INFINITY) {
    for (int s = 0; s < p.num_splits; s++) {
      float l = p.lse_part[base + (int64_t)s * r_max];
      if (l == INFINITY || l == -INFINITY) continue;         // empty split: its partial is never read
      const float w = __expf(l - m);
      tot += w;
      const h8 v = *(const h8*)(p.o_part + (base + (int64_t)s * r_max) * kDNope + lane * 8);
#pragma unroll
      for (int e = 0; e < 8; e++) a[e] += (float)v[e] * w;
    }
  }
  const float inv = tot > 0.f ? 1.f / tot : 0.f;
  __bf16* out = p.out + (int64_t)(q0 + t_local) * p.out_st + (int64_t)head * p.out_sh;
  bf16x8 o8;
#pragma unroll
  for (int e = 0; e < 8; e++) o8[e] = (__bf16)(a[e] * inv);
  *(bf16x8*)(out + lane * 8) = o8;
  if (p.lse_out && lane == 0)
    p.lse_out[(int64_t)(q0 + t_local) * p.lse_st + head] = tot > 0.f ? __logf(tot) + m : -INFINITY;
}

}  // namespace mlahip

using namespace mlahip;

extern "C" size_t mla_decode_workspace_bytes(int32_t batch, int32_t max_q_len, int32_t num_heads, int32_t num_splits) {
  if (batch <= 0 || max_q_len <= 0 || num_heads <= 0 || num_splits <= 0) return 0;
  // batch * num_splits chunks, and one more partial for every sequence boundary inside a chunk: batch * (num_splits + 1) partials in all
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * max_q_len * num_heads;
  // fp16 partials, fp32 log-sum-exps, and per row a correction record (fp32 factor + cache address)
  // ... and two partial numbers per sequence
  return rows * kDNope * sizeof(_Float16) + rows * (2 * sizeof(float) + sizeof(void*)) + (size_t)batch * 2 * sizeof(int32_t);
}

// first-generation kernel for the bf16 cache too (comparisons only)
static bool use_first_generation() {
  static const bool v = getenv("MLA_DECODE_V1") != nullptr;
  return v;
}

static int decode_split_impl(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                     int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                     int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                     int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                     const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                     const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                     int32_t max_q_len, int32_t num_heads, float scale, void* workspace,
                                     size_t workspace_bytes, int32_t num_splits, const int32_t* sparse_rows,
                                     int64_t sparse_stride, int32_t page_size, bool fp8, hipStream_t stream) {
  MLA_REQUIRE(q_nope && q_rope && nope_cache && rope_cache && (block_table || sparse_rows) && seq_lens, MLA_ERR_NULL,
              "mla_decode_bf16: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_splits >= 1 && (sparse_rows || max_blocks >= 1) &&
                  num_pages >= 1 && page_size >= 1,
              MLA_ERR_SHAPE, "mla_decode_bf16: batch=%d max_q_len=%d num_heads=%d num_splits=%d max_blocks=%d num_pages=%lld",
              batch, max_q_len, num_heads, num_splits, max_blocks, (long long)num_pages);
  MLA_REQUIRE(num_splits <= 65535 && batch <= 65535, MLA_ERR_SHAPE, "mla_decode_bf16: grid limits exceeded");
  MLA_REQUIRE((qn_stride_t % 8 == 0) && (qn_stride_h % 8 == 0) && (qr_stride_t % 8 == 0) && (qr_stride_h % 8 == 0) &&
                  (nope_row_stride % 8 == 0) && (rope_row_stride % 8 == 0) && (nope_page_stride % 8 == 0) &&
                  (rope_page_stride % 8 == 0),
              MLA_ERR_SHAPE, "mla_decode_bf16: strides must keep 16-byte alignment of 8-element groups");
  MLA_REQUIRE(((uintptr_t)q_nope % 16 == 0) && ((uintptr_t)q_rope % 16 == 0) && ((uintptr_t)nope_cache % 16 == 0) &&
                  ((uintptr_t)rope_cache % 16 == 0),
              MLA_ERR_SHAPE, "mla_decode_bf16: pointers must be 16-byte aligned");
  if (batch == 0) return MLA_OK;
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(workspace && workspace_bytes >= need, MLA_ERR_WORKSPACE,
              "mla_decode_bf16: workspace %zu bytes < required %zu", workspace_bytes, need);
  MLA_REQUIRE((uintptr_t)workspace % 16 == 0, MLA_ERR_SHAPE, "mla_decode_bf16: workspace must be 16-byte aligned");

  const int r_max = max_q_len * num_heads;
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * r_max;
  MLA_REQUIRE((int64_t)batch * num_splits <= 0x7fffffff / 2 && nope_row_stride < (1 << 28) && rope_row_stride < (1 << 28),
              MLA_ERR_SHAPE, "mla_decode_bf16: batch * num_splits or a row stride is out of range");
  DecodeParams p;
  p.q_nope = (const __bf16*)q_nope; p.qn_st = qn_stride_t; p.qn_sh = qn_stride_h;
  p.q_rope = (const __bf16*)q_rope; p.qr_st = qr_stride_t; p.qr_sh = qr_stride_h;
  p.nope = (const __bf16*)nope_cache; p.nope_sp = nope_page_stride; p.nope_sr = nope_row_stride;
  p.rope = (const __bf16*)rope_cache; p.rope_sp = rope_page_stride; p.rope_sr = rope_row_stride;
  p.block_table = block_table; p.bt_stride = bt_stride; p.max_blocks = max_blocks;
  p.seq_lens = seq_lens; p.qsl = query_start_loc;
  p.batch = batch; p.max_q_len = max_q_len; p.num_heads = num_heads; p.num_pages = num_pages;
  p.scale_log2 = scale * kLog2e;
  p.o_part = (_Float16*)workspace;
  p.lse_part = (float*)((_Float16*)workspace + rows * kDNope);
  p.num_splits = num_splits;
  p.sparse_rows = sparse_rows; p.sparse_stride = sparse_stride; p.page_size = page_size;

  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute((const void*)mla_decode_bf16_kernel<kModeDense>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeLdsB);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)mla_decode_bf16_kernel<kModeSparse>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, kDecodeLdsB);
    if (e == hipSuccess)
      e = hipFuncSetAttribute((const void*)mla_decode_bf16_kernel<kModeFp8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                              kFp8LdsB);
    if (e != hipSuccess) return fail(MLA_ERR_LAUNCH, "mla_decode_bf16: cannot reserve %d bytes of LDS: %s", kDecodeLdsB,
                                     hipGetErrorString(e));
    attr_set = true;
  }
  dim3 grid(num_splits, batch, (r_max + kRowsPerWg - 1) / kRowsPerWg);
  if (!use_first_generation()) {
    DecodeV2Params v;
    v.q_nope = p.q_nope; v.qn_st = p.qn_st; v.qn_sh = p.qn_sh; v.q_rope = p.q_rope; v.qr_st = p.qr_st; v.qr_sh = p.qr_sh;
    v.nope = p.nope; v.nope_sp = p.nope_sp; v.nope_sr = p.nope_sr; v.rope = p.rope; v.rope_sp = p.rope_sp; v.rope_sr = p.rope_sr;
    v.block_table = p.block_table; v.bt_stride = p.bt_stride; v.max_blocks = p.max_blocks; v.seq_lens = p.seq_lens; v.qsl = p.qsl;
    v.batch = p.batch; v.max_q_len = p.max_q_len; v.num_heads = p.num_heads; v.num_pages = p.num_pages;
    v.scale_log2 = p.scale_log2; v.o_part = p.o_part; v.lse_part = p.lse_part;
    v.corr_scale = p.lse_part + rows; v.corr_row = (const __bf16**)(p.lse_part + 2 * rows);
    v.seg_ids = (int32_t*)(p.lse_part + 4 * rows);
    v.sparse_rows = p.sparse_rows; v.sparse_stride = p.sparse_stride; v.page_size = p.page_size;
    v.cache8 = fp8 ? (const uint8_t*)nope_cache : nullptr; v.c8_sp = nope_page_stride;
    const dim3 grid2((unsigned)(batch * num_splits), 1, grid.z);
    if (fp8) return launch_decode_v2_fp8(v, grid2, stream);
    return launch_decode_v2(v, sparse_rows != nullptr, grid2, stream);
  }
  if (fp8) hipLaunchKernelGGL(mla_decode_bf16_kernel<kModeFp8>, grid, dim3(256), kFp8LdsB, stream, p);
  else if (sparse_rows) hipLaunchKernelGGL(mla_decode_bf16_kernel<kModeSparse>, grid, dim3(256), kDecodeLdsB, stream, p);
  else hipLaunchKernelGGL(mla_decode_bf16_kernel<kModeDense>, grid, dim3(256), kDecodeLdsB, stream, p);
  return check_launch("mla_decode_bf16_kernel");
}

// Phase 1: one normalised fp32 partial + log-sum-exp per (sequence, split, query row) into the workspace.
extern "C" int mla_decode_bf16_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                     int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                     int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                     int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                     const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                     const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                     int32_t max_q_len, int32_t num_heads, float scale, void* workspace,
                                     size_t workspace_bytes, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(block_table, MLA_ERR_NULL, "mla_decode_bf16: null block table");
  return decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                           nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                           block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads,
                           scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, false, stream);
}

// Phase 2: N-way log-sum-exp merge of the workspace partials into the bf16 output (and optional lse).
extern "C" int mla_splitkv_reduce(const void* workspace, size_t workspace_bytes, const int32_t* seq_lens,
                                  const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                  int32_t num_splits, void* out, int64_t out_stride_t, int64_t out_stride_h,
                                  float* lse_out, hipStream_t stream) {
  MLA_REQUIRE(workspace && out, MLA_ERR_NULL, "mla_splitkv_reduce: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_splits >= 1, MLA_ERR_SHAPE,
              "mla_splitkv_reduce: batch=%d max_q_len=%d num_heads=%d num_splits=%d", batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE((out_stride_t % 8 == 0) && (out_stride_h % 8 == 0) && ((uintptr_t)out % 16 == 0) &&
                  ((uintptr_t)workspace % 16 == 0),
              MLA_ERR_SHAPE, "mla_splitkv_reduce: output rows must be 16-byte aligned");
  if (batch == 0) return MLA_OK;
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(workspace_bytes >= need, MLA_ERR_WORKSPACE, "mla_splitkv_reduce: workspace %zu bytes < required %zu",
              workspace_bytes, need);
  const int r_max = max_q_len * num_heads;
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * r_max;
  if (seq_lens && !use_first_generation()) {
    // partials in chunk order, as the bf16 kernels write them
    ChunkReduceParams cp;
    cp.o_part = (const _Float16*)workspace; cp.lse_part = (const float*)((const _Float16*)workspace + rows * kDNope);
    cp.corr_scale = cp.lse_part + rows; cp.corr_row = (const __bf16* const*)(cp.lse_part + 2 * rows);
    cp.seg_ids = (const int32_t*)(cp.lse_part + 4 * rows);
    cp.seq_lens = seq_lens; cp.qsl = query_start_loc;
    cp.batch = batch; cp.max_q_len = max_q_len; cp.num_heads = num_heads; cp.num_chunks = batch * num_splits;
    cp.out = (__bf16*)out; cp.out_st = out_stride_t; cp.out_sh = out_stride_h;
    cp.lse_out = lse_out; cp.lse_st = num_heads;
    return launch_chunk_reduce(cp, stream);
  }
  ReduceParams rp;
  rp.o_part = (const _Float16*)workspace; rp.lse_part = (const float*)((const _Float16*)workspace + rows * kDNope);
  rp.qsl = query_start_loc;
  rp.batch = batch; rp.max_q_len = max_q_len; rp.num_heads = num_heads; rp.num_splits = num_splits;
  rp.out = (__bf16*)out; rp.out_st = out_stride_t; rp.out_sh = out_stride_h;
  rp.lse_out = lse_out; rp.lse_st = num_heads;
  const int64_t nrows = (int64_t)batch * r_max;
  hipLaunchKernelGGL(mla_splitkv_reduce_kernel, dim3((unsigned)((nrows + 3) / 4)), dim3(256), 0, stream, rp);
  return check_launch("mla_splitkv_reduce_kernel");
}

// Both phases on one stream.
extern "C" int mla_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                               int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                               int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                               int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                               const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                               const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                               int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                               int64_t out_stride_h, float* lse_out, void* workspace, size_t workspace_bytes,
                               int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(out, MLA_ERR_NULL, "mla_decode_bf16: null output pointer");
  int rc = mla_decode_bf16_split(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                                 nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride,
                                 num_pages, block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch,
                                 max_q_len, num_heads, scale, workspace, workspace_bytes, num_splits, stream);
  if (rc != MLA_OK) return rc;
  return mla_splitkv_reduce(workspace, workspace_bytes, seq_lens, query_start_loc, batch, max_q_len, num_heads, num_splits,
                            out, out_stride_t, out_stride_h, lse_out, stream);
}

// Sparse absorbed MLA over a per-token list of cache rows (reference: npu_sparse_flash_attention as called in
// src/omni_npu/attention/backends/dsa.py:259-291).  Token t attends to the rows sparse_rows[t, 0 .. counts[t]) that
// dsa_build_rows produced from the indexer's top-k positions.  Same split-KV kernel and reduction as the dense decode.
extern "C" int dsa_sparse_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                      int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                      int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                      int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                      int32_t page_size, const int32_t* sparse_rows, int64_t sparse_stride,
                                      const int32_t* counts, int32_t num_tokens, int32_t num_heads, float scale, void* out,
                                      int64_t out_stride_t, int64_t out_stride_h, float* lse_out, void* workspace,
                                      size_t workspace_bytes, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(sparse_rows && counts && out, MLA_ERR_NULL, "dsa_sparse_decode_bf16: null pointer argument");
  MLA_REQUIRE(sparse_stride >= 1 && page_size >= 1, MLA_ERR_SHAPE, "dsa_sparse_decode_bf16: sparse_stride=%lld page_size=%d",
              (long long)sparse_stride, page_size);
  MLA_REQUIRE(nope_page_stride == (int64_t)page_size * nope_row_stride && rope_page_stride == (int64_t)page_size * rope_row_stride,
              MLA_ERR_UNSUPPORTED, "dsa_sparse_decode_bf16: cache pages must be contiguous (page stride == page_size * row stride)");
  int rc = decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                             nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                             nullptr, 0, 0, counts, nullptr, num_tokens, 1, num_heads, scale, workspace, workspace_bytes,
                             num_splits, sparse_rows, sparse_stride, page_size, false, stream);
  if (rc != MLA_OK) return rc;
  return mla_splitkv_reduce(workspace, workspace_bytes, counts, nullptr, num_tokens, 1, num_heads, num_splits, out,
                            out_stride_t, out_stride_h, lse_out, stream);
}

// Absorbed-MLA paged decode over the fp8-e4m3 block-scaled cache written by mla_cache_write_fp8 (656-byte rows,
// row stride exactly 656, page size 128).  Tiles are dequantised to bf16 in LDS and then take the bf16 MFMA path, so
// the arithmetic is "dequantise, then attend" as in the CPU restatement.  The reference has no fp8 cache
// (src/omni_npu/attention/backends/mla.py:791-792 passes antiquant_mode=0, antiquant_scale=None).
extern "C" int mla_decode_fp8(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                              int64_t qr_stride_t, int64_t qr_stride_h, const void* cache, int64_t page_stride_bytes,
                              int64_t row_stride_bytes, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                              int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                              int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                              int64_t out_stride_h, float* lse_out, void* workspace, size_t workspace_bytes,
                              int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(cache && out && block_table, MLA_ERR_NULL, "mla_decode_fp8: null pointer argument");
  MLA_REQUIRE(row_stride_bytes == kFp8RowB && page_stride_bytes >= (int64_t)kPage * kFp8RowB && page_stride_bytes % 16 == 0,
              MLA_ERR_UNSUPPORTED, "mla_decode_fp8: rows must be exactly 656 bytes apart, pages 128 rows (got %lld / %lld)",
              (long long)row_stride_bytes, (long long)page_stride_bytes);
  // the shared validation wants element strides that are multiples of 8: hand it byte strides that are
  int rc = decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, cache, page_stride_bytes,
                             kFp8RowB + 8 /* unused in fp8 mode */, cache, page_stride_bytes, kFp8RowB + 8, num_pages,
                             block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads,
                             scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, true, stream);
  if (rc != MLA_OK) return rc;
  // the first-generation kernel writes its partials in [sequence][split] order (no sequence lengths, no chunk arithmetic),
  // the current one in the balanced chunk order of the bf16 path
  return mla_splitkv_reduce(workspace, workspace_bytes, use_first_generation() ? nullptr : seq_lens, query_start_loc, batch,
                            max_q_len, num_heads, num_splits, out, out_stride_t, out_stride_h, lse_out, stream);
}
