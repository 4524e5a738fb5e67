// Absorbed-MLA paged decode over the fp8-e4m3 block-scaled latent cache (656-byte rows: 512 fp8 | 4 fp32 scales, one per
// 128 elements | 64 bf16 rope), second-generation kernel.
//
// Same structure as mla_decode_v2_kernel (decode_v2.hip: d-sliced P.V, fixed-reference softmax, balanced chunks, fp16
// partials merged by mla_chunk_reduce_kernel); what differs is how a block reaches the bf16 tile the MFMA phases read:
//   * the first 528 bytes of each of the block's 32 rows are copied global -> LDS as they are (two raw stages of
//     16.5 KiB), the rope part goes straight into the rope buffers (it is bf16 already);
//   * at the top of body i all 256 threads turn raw block i+2 into bf16 (x = e4m3 * block scale, rounded to bf16:
//     "dequantise, then attend") in one of THREE 32 KiB tile buffers, in the swizzled layout of the bf16 kernel;
//   * the copies of block i+3 are issued right after.
// LDS: 3 x 32 KiB tiles + 3 x 4 KiB rope + 2 x 17 KiB raw + 16 KiB P exchange + flags = 159 KiB.
// The dominant-key correction of the bf16 kernel is not applied (its record would have to name a bf16 row); the fp8 cache
// has a wider error budget.  No reference counterpart: src/omni_npu/attention/backends/mla.py:791-792 passes
// antiquant_mode=0, antiquant_scale=None.
#include "decode_v2_params.hpp"
#include <type_traits>
#include <cstdlib>

namespace mlahip {
namespace f8v2 {

#ifndef MLA_V2_QK_AHEAD
#define MLA_V2_QK_AHEAD 4
#endif
#ifndef MLA_V2_PV_AHEAD
#define MLA_V2_PV_AHEAD 2
#endif
constexpr int kQkAheadV2 = MLA_V2_QK_AHEAD, kPvAheadV2 = MLA_V2_PV_AHEAD;   // LDS read-ahead depth, in fragments
constexpr int kBlk = 32;                                   // tokens per block
constexpr int kV2NopeBufB = kBlk * 1024;                   // 32768
constexpr int kV2RopeBufB = kBlk * 128;                    // 4096
constexpr int kV2RopeOff = 3 * kV2NopeBufB;                // 98304 (three tile buffers)
constexpr int kRawRowB = 528;                              // staged bytes of a 656-byte row: fp8 latent + scales
constexpr int kRawStageB = 17 * 1024;                       // 32 rows x 528 B = 16896, padded to 17 copy instructions
constexpr int kRawOff = kV2RopeOff + 3 * kV2RopeBufB;      // 110592
constexpr int kRawGranules = kBlk * kRawRowB / 16;         // 1056
constexpr int kFp8RowBytes = 656, kFp8RopeOffB = 528;
constexpr int kV2POff = kRawOff + 2 * kRawStageB;          // 145408
constexpr int kV2PBufB = 8192;                             // 4 row groups x 2 k-blocks x 64 lanes x 16 B
constexpr int kV2AOff = kV2POff + 2 * kV2PBufB;            // 161792: restart flags, 2 x 512 B
constexpr int kV2LdsB = kV2AOff + 2 * 512;                 // 162816
#ifndef MLA_V2_LEAD
#define MLA_V2_LEAD 3
#endif
constexpr int kLead = MLA_V2_LEAD;                          // block i + kLead is copied while block i is consumed (2 or 3)
constexpr float kRestartThreshold = 100.f;                 // log2 units above a row's reference

__device__ __forceinline__ int v2_swz_nope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r1 ^ r3) << 3) | (r0 << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int v2_swz_rope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r0 ^ r3) << 2) | (r1 << 1) | r2;
}


// value of the same lane index in the other half of the wavefront, combined with max / add (one VALU swap, no LDS)
__device__ __forceinline__ float half_max(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ int half_max_i32(int v) {
  const auto r = __builtin_amdgcn_permlane32_swap((uint32_t)v, (uint32_t)v, false, false);
  return max((int)r[0], (int)r[1]);
}
__device__ __forceinline__ float half_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

__device__ __forceinline__ int v2_num_blocks(int len) { return len > 0 ? (len + kBlk - 1) / kBlk : 0; }
constexpr int kSegCost = 8;                                // start-up cost of a segment, in blocks (about 19 us / 2.3 us)
__device__ __forceinline__ int v2_work_units(int len) { return len > 0 ? (len + kBlk - 1) / kBlk + kSegCost : 0; }
static_assert(kBlk == kPlanBlk && kSegCost == kPlanSegCost, "the merge kernels recompute the chunk plan with these constants");
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}
__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v = max(v, __shfl_xor(v, d, 64));
  return v;
}
__device__ __forceinline__ int wave_incl_scan_i32(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) { const int t = __shfl_up(v, d, 64); v += lane >= d ? t : 0; }
  return v;
}

typedef __attribute__((address_space(4))) const int32_t* ConstI32Ptr;   // scalar (constant-cache) loads

// kWindow: static sink keys followed by a sliding window, as in the bf16 kernel: the sequence is walked without the
// blocks between the sink and the window (block v at or behind the first non-sink block is block v + skip of the cache),
// and the blocks right behind the sink mask the keys older than a row's window.
template <bool kWindow>
__global__ __launch_bounds__(256, 1) void mla_decode_v2_fp8_kernel(const DecodeV2Params p) {
  constexpr bool kSparse = false;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h32 = lane & 31;
  const int half = lane >> 5;
  // The row groups of one chunk (more than 128 query rows: several tokens per sequence) stream the same cache rows.
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has its own L2, so they are renumbered to
  // sit on one XCD, next to each other in its queue: they run at the same time and share the rows in that L2.
  int chunk = blockIdx.x, grp = blockIdx.z;
  if (gridDim.z > 1 && (gridDim.x & 7) == 0) {
    const int lin = blockIdx.x + gridDim.x * blockIdx.z;
    const int j = lin >> 3;
    grp = j % gridDim.z;
    chunk = (j / gridDim.z) * 8 + (lin & 7);
  }
  const int r_max = p.max_q_len * p.num_heads;
  if (grp * 128 >= r_max) return;
  const uint32_t lds0 = lds_addr_of(lds);

  // ---- which blocks are mine ----
  // Work is measured in units of one 32-token block; starting a segment (query load, first copies, epilogue, partial
  // write) costs about kSegCost of them.  Every non-empty sequence is laid out as kSegCost units of start-up followed by
  // its blocks, the sequences end to end, and that line is cut into gridDim.x chunks of equal length: chunk c covers
  // units [c*T/G, (c+1)*T/G), and a chunk that holds the start of a sequence gets that many fewer blocks.  A chunk that
  // crosses a sequence boundary is processed as two (or more) segments; the segment of sequence b in chunk c writes
  // partial number c + b, so the partials of one sequence are consecutive and mla_chunk_reduce_kernel finds them with
  // the same arithmetic.  Every wavefront derives the plan by itself from the sequence lengths (two passes: total, scan).
  int seg_b;
  int64_t v_cur, v_end, v_seq;                                // my units [v_cur, v_end); first unit of sequence seg_b + 1
  {
    int tot = 0;
    for (int i = lane; i < p.batch; i += 64) tot += v2_work_units(p.seq_lens[i]);
    tot = __builtin_amdgcn_readfirstlane(wave_sum_i32(tot));
    const int64_t cb = (int64_t)chunk * tot / gridDim.x, ce = (int64_t)(chunk + 1) * tot / gridDim.x;
    if (cb == ce) return;
    int carry = 0, b0 = 0, pb0 = 0;
    for (int base = 0; base < p.batch; base += 64) {
      const int i = base + lane;
      const int c = i < p.batch ? v2_work_units(p.seq_lens[i]) : 0;
      const int pe = wave_incl_scan_i32(c, lane) + carry;     // units of sequences 0..i
      const bool le = i < p.batch && pe <= cb;                // sequence i ends at or before my first unit
      b0 += __builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
      pb0 = max(pb0, wave_max_i32(le ? pe : 0));
      carry = __builtin_amdgcn_readlane(pe, 63);
    }
    seg_b = __builtin_amdgcn_readfirstlane(b0) - 1;
    v_seq = __builtin_amdgcn_readfirstlane(pb0);
    v_cur = cb;
    v_end = ce;
  }

  while (v_cur < v_end) {
  seg_b++;
  if (seg_b >= p.batch) break;
  const int b = seg_b;
  const int L = p.seq_lens[b];
  const int64_t v_b = v_seq;                                  // first unit of sequence b
  v_seq += v2_work_units(L);
  const int64_t v_hi = v_seq < v_end ? v_seq : v_end;
  int blk_begin = (int)(v_cur - v_b) - kSegCost;
  int blk_end = (int)(v_hi - v_b) - kSegCost;
  blk_begin = blk_begin < 0 ? 0 : blk_begin;
  blk_end = blk_end < 0 ? 0 : blk_end;
  v_cur = v_hi;
  const int nb = blk_end - blk_begin;
  if (nb <= 0) continue;
  // the merge kernel finds the partials of a sequence between the numbers its first and its last segment leave here
  if (threadIdx.x == 0) {
    if (blk_begin == 0) p.seg_ids[2 * b] = chunk + b;
    if (blk_end == v2_num_blocks(L)) p.seg_ids[2 * b + 1] = chunk + b;
  }
  lds_barrier();                                              // the previous segment's epilogue is done with the buffers

  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  qlen = qlen < p.max_q_len ? qlen : p.max_q_len;
  const int rows = qlen * p.num_heads;

  // this lane's query row for QK / softmax (row group = wave)
  const int row = grp * 128 + wave * 32 + h32;
  const bool row_ok = row < rows && L > 0;
  const int t_local = row / p.num_heads;
  const int head = row - t_local * p.num_heads;
  int limit = row_ok ? (L - qlen + t_local + 1) : 0;         // keys [0, limit) are visible to this row
  limit = limit < 0 ? 0 : limit;
  const int win_skip = kWindow ? p.win_skip[b] : 0;
  const int win_blk0 = kWindow ? p.win_sink / kBlk : 0;
  const int64_t part_base = (int64_t)(chunk + b) * r_max + grp * 128;   // + row index in the group

  if (grp * 128 >= rows) {
    if (row < r_max && half == 0) { p.lse_part[part_base + wave * 32 + h32] = -INFINITY; p.corr_scale[part_base + wave * 32 + h32] = 0.f; }
    continue;
  }

  // ---- global -> LDS copies: the first 528 bytes of the block's 32 rows land row after row in a raw stage (1056 granules of
  // 16 bytes = 16.5 instructions of 64 lanes: five per wave, the tail lanes idle), the rope part of every row goes to
  // the rope buffer (one instruction of 8 rows per wave, swizzled by the copying lane).  Rows past the end of the
  // sequence re-read its last row (their scores are masked; their bytes must be finite).
  const uint32_t rope_off = (uint32_t)(((lane & 7) ^ v2_swz_rope((wave * 8 + (lane >> 3)) & 15)) << 4);
  const uint32_t rope_voff = (uint32_t)(wave * 8 + (lane >> 3)) * kFp8RowBytes + kFp8RopeOffB + rope_off;   // full blocks
  // instruction k (0..16) of a block copies granules 64k..64k+63 and belongs to wave k % 4; the last one is half
  // empty: its upper lanes copy granule 1055 again, into the padding of the stage
  uint32_t raw_voff[5];                                       // full blocks: source offset of my granule of my j-th instruction
#pragma unroll
  for (int j = 0; j < 5; j++) {
    int gi = (wave + 4 * j) * 64 + lane;
    gi = gi < kRawGranules ? gi : kRawGranules - 1;
    const int r = gi / 33, g = gi - r * 33;
    raw_voff[j] = (uint32_t)(r * kFp8RowBytes + g * 16);
  }
  ConstI32Ptr bt = (ConstI32Ptr)(p.block_table) + (int64_t)b * p.bt_stride;
  auto load_page = [&](int page) -> int64_t {
    page = page < p.max_blocks ? page : p.max_blocks - 1;
    int64_t pg = bt[page];
    return pg < 0 ? 0 : (pg >= p.num_pages ? p.num_pages - 1 : pg);
  };
  // The page of the block being copied and the next one are kept in scalar registers, so the block-table load is never
  // waited for in the loop (blocks are requested in ascending order; a restart begins again at the first block)
  int page_cur = -1;
  int64_t pg_cur = 0, pg_nxt = 0;
  auto issue_block = [&](int blk) {
    const int last = L - 1 - blk * kBlk;                      // last valid row of the block (>= 0)
    const uint32_t raw = lds0 + kRawOff + (blk & 1) * kRawStageB;
    const uint32_t rbuf = lds0 + kV2RopeOff + (blk % 3) * kV2RopeBufB;
    const int cblk = blk + (kWindow && blk >= win_blk0 ? win_skip : 0);   // block of the cache
    const int page = cblk >> 2;
    if (blk == blk_begin) { page_cur = page; pg_cur = load_page(page); pg_nxt = load_page(page + 1); }
    else if (page != page_cur) {
      pg_cur = (kWindow && page != page_cur + 1) ? load_page(page) : pg_nxt;   // the jump from the sink to the window
      page_cur = page;
      pg_nxt = load_page(page + 1);
    }
    const char* src = (const char*)p.cache8 + pg_cur * p.c8_sp + (int64_t)(cblk & 3) * kBlk * kFp8RowBytes;
    if (last >= kBlk - 1) {
#pragma unroll
      for (int j = 0; j < 5; j++)
        if (wave + 4 * j < 17) dma16_sv(src, raw_voff[j], __builtin_amdgcn_readfirstlane(raw + (wave + 4 * j) * 1024));
      dma16_sv(src, rope_voff, __builtin_amdgcn_readfirstlane(rbuf + wave * 1024));
    } else {
#pragma unroll
      for (int j = 0; j < 5; j++) {
        int gi = (wave + 4 * j) * 64 + lane;
        gi = gi < kRawGranules ? gi : kRawGranules - 1;
        const int r = gi / 33, g = gi - r * 33;
        const int re = r < last ? r : last;
        if (wave + 4 * j < 17) dma16_sv(src, (uint32_t)(re * kFp8RowBytes + g * 16), __builtin_amdgcn_readfirstlane(raw + (wave + 4 * j) * 1024));
      }
      const int r = wave * 8 + (lane >> 3);
      const int re = r < last ? r : last;
      dma16_sv(src, (uint32_t)(re * kFp8RowBytes + kFp8RopeOffB) + rope_off, __builtin_amdgcn_readfirstlane(rbuf + wave * 1024));
    }
  };
  // raw block `blk` -> bf16 tile buffer blk % 3, all 256 threads: thread (row r, chunk c) turns 16 e4m3 values into two
  // 16-byte granules of the swizzled row
  // Thread t owns row t/8 and the 16-element chunks t%8 + 8*it (it = 0..3: one per scale block), so that every address is
  // one of two per-thread bases plus a compile-time offset (the swizzle only touches the low four granule bits).
  const int dq_row = (int)threadIdx.x >> 3, dq_c0 = (int)threadIdx.x & 7;
  const uint32_t dq_src = (uint32_t)(kRawOff + dq_row * kRawRowB + dq_c0 * 16);
  const uint32_t dq_dst0 = (uint32_t)(dq_row * 1024 + (((2 * dq_c0) ^ v2_swz_nope(dq_row & 15)) << 4));
  const uint32_t dq_dst1 = (uint32_t)(dq_row * 1024 + (((2 * dq_c0 + 1) ^ v2_swz_nope(dq_row & 15)) << 4));
  auto dequant_block = [&](int blk) {
    const char* raw = lds + (blk & 1) * kRawStageB + dq_src;
    char* tile = lds + (blk % 3) * kV2NopeBufB;
    const f32x4 sc4 = *(const f32x4*)(lds + kRawOff + (blk & 1) * kRawStageB + dq_row * kRawRowB + 512);
#pragma unroll
    for (int it = 0; it < 4; it++) {
      const u32x4 w = *(const u32x4*)(raw + it * 128);
      const float sc = sc4[it];
      u32x4 lo, hi;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x2 x0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], false);
        const f32x2 x1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], true);
        bf16x2 y0, y1;
        y0[0] = (__bf16)(x0[0] * sc); y0[1] = (__bf16)(x0[1] * sc);
        y1[0] = (__bf16)(x1[0] * sc); y1[1] = (__bf16)(x1[1] * sc);
        const uint32_t p0 = __builtin_bit_cast(uint32_t, y0), p1 = __builtin_bit_cast(uint32_t, y1);
        if (j < 2) { lo[2 * j] = p0; lo[2 * j + 1] = p1; } else { hi[2 * (j - 2)] = p0; hi[2 * (j - 2) + 1] = p1; }
      }
      *(u32x4*)(tile + dq_dst0 + it * 256) = lo;
      *(u32x4*)(tile + dq_dst1 + it * 256) = hi;
    }
  };

  // ---- prologue: the first block's copies go out, then the query loads; both are waited for together ----
  issue_block(blk_begin);
  bf16x8 qf[36];
  {
    // All 36 loads go out back to back and are waited for once (written as assembly: the compiler, short of registers,
    // would wait for each load before issuing the next).  Rows that do not exist read row 0 of the sequence instead:
    // their results are finite and never stored.
    const int64_t tq = row_ok ? (q0 + t_local) : q0;
    const int64_t hq = row_ok ? head : 0;
    const __bf16* qn = p.q_nope + tq * p.qn_st + hq * p.qn_sh + half * 8;
    const __bf16* qr = p.q_rope + tq * p.qr_st + hq * p.qr_sh + half * 8;
#pragma unroll
    for (int kk = 0; kk < 32; kk++) asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(qf[kk]) : "v"(qn), "i"(kk * 32));
#pragma unroll
    for (int kk = 0; kk < 4; kk++) asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "=v"(qf[32 + kk]) : "v"(qr), "i"(kk * 32));
    // (a builtin, so that the compiler's own bookkeeping of outstanding loads is cleared too: otherwise it would guard
    // the first use of any earlier load inside the main loop with a full wait, on every iteration)
    __builtin_amdgcn_s_waitcnt(0x0F70);                                         // vmcnt(0)
#pragma unroll
    for (int kk = 0; kk < 36; kk++) asm volatile("" : "+v"(qf[kk]));           // the query stays in VGPRs
  }

  f32x16 acc[4][4];                                          // [d block of this wave's slice][row group]
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  float m_ref = -INFINITY;       // this row's softmax reference (log2 domain), fixed once finite
  float m_seen = -INFINITY;      // largest score seen so far (reference of a restart)
  float l_run = 0.f;

  // ---- per-lane LDS offsets ----
  // The swizzles are XORs confined to bits 4..7 of a byte offset whose other low bits are zero, so one base register
  // per access pattern plus an XOR with a compile-time constant reaches every fragment (registers are the scarce
  // resource here: a single spilled value would be reloaded with a vector-memory wait that also waits for the LDS copies).
  const int fk = v2_swz_nope(h32 & 15), fr = v2_swz_rope(h32 & 15);
  const uint32_t kbase = (uint32_t)(h32 * 1024 + ((half ^ fk) << 4));                 // ^ (j << 5), + (kk/8)*256, + buffer
  const uint32_t rbase = (uint32_t)(kV2RopeOff + h32 * 128 + ((half ^ fr) << 4));     // ^ (j << 5), + buffer
  const int g16 = lane >> 4, j16 = lane & 15;
  const int v_row = 4 * (g16 >> 1) + (j16 >> 2);              // + 8*rd + 16*kb
  const int v_cl = 2 * (g16 & 1) + ((j16 & 3) >> 1);
  const int v_in = (j16 & 1) * 8;
  uint32_t vbase[2];                                          // [rd]: ^ (db << 6), + kb*16384, + buffer
#pragma unroll
  for (int rd = 0; rd < 2; rd++) {
    const int rr = v_row + 8 * rd;
    vbase[rd] = (uint32_t)(rr * 1024 + v_in + wave * 256 + ((v_cl ^ v2_swz_nope(rr & 15)) << 4));
  }
  // P^T fragments and restart flags in LDS.  These offsets are recomputed from the hardware lane number wherever they are
  // used instead of living in registers across the loop: every register counts (a spilled value would be reloaded with
  // a vector-memory wait that also waits for the copies in flight).
  auto lane_now = [] { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); };
  auto p_w_off = [&] { return kV2POff + (wave * 2 * 64 + lane_now()) * 16; };   // + kb*1024 + parity*8192: this wave's fragments
  auto p_r_off = [&] { return kV2POff + lane_now() * 16; };                     // + (rg*2 + kb)*1024 + parity*8192
  auto a_r_off = [&] { return kV2AOff + (lane_now() & 31) * 16; };              // + parity*512: flags of rows (rg, h32), 4 floats
  auto a_w_off = [&] { return kV2AOff + (lane_now() & 31) * 16 + wave * 4; };

  // S^T for block `blk`.  The K fragments are read with hand-placed LDS instructions, kQkAheadV2 fragments ahead of the
  // MFMA that consumes them, and explicit lgkmcnt waits: left to itself the compiler funnels every fragment through one
  // register quad and waits for each read in full, which exposes the whole LDS latency 36 times per block.  (LDS reads
  // return in order, so compiler-issued reads around this section only make its own waits stricter, never wrong.)
  // The MFMAs of this phase are written as assembly with the scores in ordinary vector registers: the compiler would
  // put every MFMA result into the accumulation file, which is full of output accumulators, and shuffle 48 registers
  // per block to make room.  Hazards the compiler would otherwise pad: none between dependent MFMAs of one shape with
  // identical C and D; the wait after the last one (MFMA result read by the vector ALU) is the s_nop pair at the end.
  // With kIssue the nine copies of block `blk_issue` are spread over the MFMAs.
  auto qk_block = [&](int blk, f32x16& s, auto issue, int blk_issue, auto&& mid_hook) {
    constexpr int kIssueMode = decltype(issue)::value;       // 0: no copies; 1: any block; 2: a full block of the paged cache
    constexpr bool kIssue = kIssueMode != 0;
    const uint32_t nb32 = lds0 + (blk % 3) * kV2NopeBufB + kbase;     // buffers are 4 KiB aligned: the XORs below stay exact
    const uint32_t rb32 = lds0 + (blk % 3) * kV2RopeBufB + rbase;
    bf16x8 ka[kQkAheadV2];
#define MLA_K_READ(dst, kk)                                                                                         \
    do {                                                                                                            \
      if ((kk) < 32) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(nb32 ^ (uint32_t)(((kk) & 7) << 5)), "i"(((kk) >> 3) * 256)); \
      else asm volatile("ds_read_b128 %0, %1" : "=v"(dst) : "v"(rb32 ^ (uint32_t)(((kk) & 3) << 5)));              \
    } while (0)
#pragma unroll
    for (int i = 0; i < kQkAheadV2; i++) MLA_K_READ(ka[i], i);
#pragma unroll
    for (int kk = 0; kk < 36; kk++) {
      // wait until fragment kk has landed: at most min(kQkAheadV2 - 1, 35 - kk) younger reads may still be in flight
      constexpr int D = kQkAheadV2;
      const int younger = (36 - 1 - kk) < (D - 1) ? (36 - 1 - kk) : (D - 1);
      if (younger >= 7) asm volatile("s_waitcnt lgkmcnt(7)" : "+v"(ka[kk % D]));
      else if (younger == 6) asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(ka[kk % D]));
      else if (younger == 5) asm volatile("s_waitcnt lgkmcnt(5)" : "+v"(ka[kk % D]));
      else if (younger == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(ka[kk % D]));
      else if (younger == 3) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(ka[kk % D]));
      else if (younger == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(ka[kk % D]));
      else if (younger == 1) asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(ka[kk % D]));
      else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ka[kk % D]));
      if (kk == 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(s) : "v"(ka[kk % D]), "v"(qf[kk]));
      else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(s) : "v"(ka[kk % D]), "v"(qf[kk]));
      if (kk + D < 36) MLA_K_READ(ka[kk % D], kk + D);
      if (kk == 27) mid_hook();
    }
#undef MLA_K_READ
    asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s));
  };

  // Softmax of block `blk` from raw scores s, cut into eight straight-line steps so that it can be interleaved with the
  // P.V MFMAs of the previous block (step k is called after the k-th group of four MFMAs; the MFMAs run 32 clocks each
  // while the vector ALU is otherwise idle).  The row maximum is taken over all 32 scores of the block, visible or not:
  // it only serves as a reference, and any finite reference within 2^100 of the true maximum is as good as another.
  struct SoftmaxState { float neg_ref, flag; bf16x8 pb[2]; float psum; };
  auto softmax_step = [&](int step, f32x16& s, SoftmaxState& st) {
    if (step == 0) {
      float mx = fmaxf(s[0], s[1]);
#pragma unroll
      for (int r = 2; r < 16; r += 2) mx = fmaxf(mx, fmaxf(s[r], s[r + 1]));
      const float mx_raw = half_max(mx);
      mx = mx_raw * p.scale_log2;
      m_seen = fmaxf(m_seen, mx);
      if (m_ref == -INFINITY) m_ref = mx;                    // the first block fixes the reference
      st.flag = mx > m_ref + kRestartThreshold ? -1.f : 1.f; // -1 asks the workgroup to restart with better references
      st.neg_ref = -m_ref;
      st.psum = 0.f;
    } else if (step <= 4) {
#pragma unroll
      for (int r = 4 * (step - 1); r < 4 * step; r++) {
        // an overflow to +inf can only happen past the restart threshold, and a restart discards everything accumulated
        s[r] = fast_exp2(__builtin_fmaf(s[r], p.scale_log2, st.neg_ref));
        st.psum += s[r];
      }
    } else if (step == 5) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int e = 0; e < 8; e++) st.pb[kb][e] = (__bf16)s[kb * 8 + e];
    }
  };
  // After the steps: the last blocks of a sequence hold keys that some rows must not see (causal multi-token queries,
  // rows past the end of the sequence); only those blocks pay for the masking.  Then P^T and the flag go to LDS.
  auto softmax_finish = [&](int blk, f32x16& s, SoftmaxState& st) {
    bool front = false;                                       // window: a block with keys older than some row's window
    if constexpr (kWindow) front = blk >= win_blk0 && blk * kBlk < L - p.win_size;
    if ((blk + 1) * kBlk > L - p.max_q_len + 1 || front) {
      int blk_s = blk;                                        // opaque: keeps the compiler from carrying `rel` as a loop
      asm volatile("" : "+s"(blk_s));                         // variable of its own (one more register across the loop)
      const int rel = limit - blk_s * kBlk - ((lane_now() >> 3) & 4);   // score r is visible iff 8*(r/4) + r%4 < rel
      // ... and, behind the sink, iff it is one of the row's newest win_size keys: 8*(r/4) + r%4 >= rel - win_size
      const int rel_lo = (kWindow && blk >= win_blk0) ? rel - p.win_size : -64;
      st.psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int kpos = 8 * (r >> 2) + (r & 3);
        s[r] = (kpos < rel && kpos >= rel_lo) ? s[r] : 0.f;
        st.psum += s[r];
      }
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int e = 0; e < 8; e++) st.pb[kb][e] = (__bf16)s[kb * 8 + e];
    }
    l_run += st.psum;
    char* base = lds + (blk & 1) * kV2PBufB;
    const int pw = p_w_off();
    *(bf16x8*)(base + pw) = st.pb[0];
    *(bf16x8*)(base + pw + 1024) = st.pb[1];
    if (lane_now() < 32) *(float*)(lds + (blk & 1) * 512 + a_w_off()) = st.flag;
  };

  // O^T += V^T P^T for block `blk`: this wave's 128 output columns for all four row groups; with kFused the softmax of
  // block blk+1 (scores s) rides along
  // First operands of the P.V phase of block `blk`, read with hand-placed instructions from inside the QK phase (they do
  // not depend on it), so that the first P.V MFMA finds them in registers.
  struct PvHead { bf16x8 pr[4]; bf16x4 v[4]; };
  auto pv_head_read = [&](int blk, PvHead& h) {
    const uint32_t pb32 = lds0 + (blk & 1) * kV2PBufB + p_r_off();
    const uint32_t vb32 = lds0 + (blk % 3) * kV2NopeBufB;
#pragma unroll
    for (int rg = 0; rg < 4; rg++) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(h.pr[rg]) : "v"(pb32), "i"(rg * 2 * 1024));
#pragma unroll
    for (int j = 0; j < 2; j++) {
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(h.v[2 * j]) : "v"(vb32 + (vbase[0] ^ (uint32_t)(j << 6))));
      asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(h.v[2 * j + 1]) : "v"(vb32 + (vbase[1] ^ (uint32_t)(j << 6))));
    }
  };
  auto pv_head_wait = [&](PvHead& h) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(h.pr[0]), "+v"(h.pr[1]), "+v"(h.pr[2]), "+v"(h.pr[3]), "+v"(h.v[0]), "+v"(h.v[1]),
                 "+v"(h.v[2]), "+v"(h.v[3]));
  };
  auto pv_block = [&](int blk, auto fused, f32x16& s, SoftmaxState& st, auto preloaded, PvHead& head) {
    constexpr bool kFused = decltype(fused)::value;
    constexpr bool kPre = decltype(preloaded)::value;
    static_assert(kPvAheadV2 == 2, "the preloaded head holds two V^T fragments");
    const char* pbase = lds + (blk & 1) * kV2PBufB;
    const char* vb = lds + (blk % 3) * kV2NopeBufB;
    auto v_frag = [&](int stp) -> bf16x8 {                    // stp = 4*kb + db
      const int db = stp & 3, kb = stp >> 2;
      bf16x4 lo = lds_read_tr16(vb + kb * 16 * 1024 + (vbase[0] ^ (uint32_t)(db << 6)));
      bf16x4 hi = lds_read_tr16(vb + kb * 16 * 1024 + (vbase[1] ^ (uint32_t)(db << 6)));
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    bf16x8 va[kPvAheadV2];
    if constexpr (kPre) {
      pv_head_wait(head);
#pragma unroll
      for (int j = 0; j < 2; j++) va[j] = __builtin_shufflevector(head.v[2 * j], head.v[2 * j + 1], 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
#pragma unroll
      for (int j = 0; j < kPvAheadV2; j++) va[j] = v_frag(j);
    }
#pragma unroll
    for (int kb = 0; kb < 2; kb++) {
      bf16x8 pr[4];
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        if (kPre && kb == 0) pr[rg] = head.pr[rg];
        else pr[rg] = *(const bf16x8*)(pbase + p_r_off() + (rg * 2 + kb) * 1024);
      }
#pragma unroll
      for (int db = 0; db < 4; db++) {
        const int stp = kb * 4 + db;
        const bf16x8 a = va[stp % kPvAheadV2];
        if (stp + kPvAheadV2 < 8) va[stp % kPvAheadV2] = v_frag(stp + kPvAheadV2);
#pragma unroll
        for (int rg = 0; rg < 4; rg++)
          acc[db][rg] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pr[rg], acc[db][rg], 0, 0, 0);
        if constexpr (kFused) softmax_step(stp, s, st);
      }
    }
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) asm volatile("" : "+a"(acc[db][rg]));     // output accumulators stay in AGPRs
  };
  // every wave reads the same 128 flags: a uniform decision.  The read is issued right after the barrier and tested after
  // the QK phase, when it has long landed; acting late is harmless because a restart discards everything.
  auto flags_read = [&](int blk) -> f32x4 { return *(const f32x4*)(lds + (blk & 1) * 512 + a_r_off()); };
  auto flags_ask_restart = [&](const f32x4& fl) -> bool {
    return __builtin_amdgcn_ballot_w64(fl[0] < 0.f || fl[1] < 0.f || fl[2] < 0.f || fl[3] < 0.f) != 0;
  };

  bool restart = false;
  do {
    if (restart) {
      // a row outgrew its reference: drain, take the maxima seen so far as references, clear the sums, start over
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      m_ref = m_seen;
      l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
      issue_block(blk_begin);
      MLA_WAIT_VMCNT(0);
      restart = false;
    }
    // ---- start-up: raw block 0 has landed (this wave's part; the barrier covers the others) ----
    if (nb > 1) issue_block(blk_begin + 1);                   // raw stage 1, rope buffer 1
    lds_barrier();
    dequant_block(blk_begin);                                 // raw stage 0 -> tile 0
    MLA_WAIT_VMCNT(0);
    lds_barrier();                                            // tile 0 complete, raw block 1 landed, stage 0 free
    if (nb > 1) dequant_block(blk_begin + 1);                 // raw stage 1 -> tile 1 (read after the next barrier)
    if (nb > 2) issue_block(blk_begin + 2);                   // raw stage 0, rope buffer 2
    // ---- block 0: QK, softmax, publish ----
    {
      f32x16 s;
      SoftmaxState st;
      qk_block(blk_begin, s, std::integral_constant<int, 0>{}, 0, [] {});
#pragma unroll
      for (int step = 0; step < 7; step++) softmax_step(step, s, st);
      softmax_finish(blk_begin, s, st);
    }
    // Everything the loop keeps in registers is touched here: a value that was parked in scratch during the prologue is
    // brought back (and waited for) now, not at its first use inside the loop, where the wait would recur every iteration
    // and stall on the copies in flight.
    asm volatile("" :: "v"(limit), "v"(kbase), "v"(rbase), "v"(vbase[0]), "v"(vbase[1]), "v"(m_ref), "v"(m_seen), "v"(l_run),
                 "v"(dq_src), "v"(dq_dst0), "v"(dq_dst1), "v"(raw_voff[0]), "v"(raw_voff[1]), "v"(raw_voff[2]), "v"(raw_voff[3]),
                 "v"(raw_voff[4]), "v"(rope_voff));
    // ---- steady state: dequantise block i+2, request block i+3, QK(i+1), then P.V(i) with the softmax of block i+1 ----
    for (int i = 0; i + 1 < nb; i++) {
      const int blk = blk_begin + i;
      // tile i+1 is complete, raw block i+2 has landed, P(i) is published, everyone is done with P.V(i-1) (tile (i+2)%3)
      // and with raw stage (i+1)&1
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      const f32x4 fl = flags_read(blk);
      if (i + 2 < nb) dequant_block(blk + 2);
      if (i + 3 < nb) issue_block(blk + 3);
      f32x16 s;
      PvHead head;
      auto hook = [&] { pv_head_read(blk, head); };
      qk_block(blk + 1, s, std::integral_constant<int, 0>{}, 0, hook);
      if (flags_ask_restart(fl)) { restart = true; break; }
      SoftmaxState st;
      pv_block(blk, std::true_type{}, s, st, std::true_type{}, head);
      softmax_finish(blk + 1, s, st);
    }
    if (!restart) {
      const int blk = blk_end - 1;
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      if (flags_ask_restart(flags_read(blk))) restart = true;
      else { f32x16 s; SoftmaxState st; PvHead head; pv_block(blk, std::false_type{}, s, st, std::false_type{}, head); }
    }
  } while (restart);

  // ---- epilogue ----
  lds_barrier();                                              // all PV done; tile buffers and P buffers are free
  {
    const float l_tot = half_sum(l_run);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const float corr = 0.f;                                   // no dominant-key correction over the fp8 cache
    const __bf16* vrow = nullptr;
    if (half == 0) {
      *(float*)(lds + kV2POff + h32 * 16 + wave * 4) = inv;
      if (row < r_max) {
        const int64_t pr = part_base + wave * 32 + h32;
        p.lse_part[pr] = l_tot > 0.f ? (m_ref + fast_log2(l_tot)) * kLn2 : -INFINITY;
        p.corr_scale[pr] = corr;
        p.corr_row[pr] = vrow;
      }
    }
  }
  lds_barrier();
  const f32x4 inv4 = *(const f32x4*)(lds + kV2POff + h32 * 16);
  // transpose through this wave's private 32 KiB (nope buffer `wave`): two rounds of 64 rows x 128 columns, fp16
  char* stage = lds + wave * kV2NopeBufB;
#pragma unroll
  for (int round = 0; round < 2; round++) {
#pragma unroll
    for (int rgl = 0; rgl < 2; rgl++) {
      const int rg = round * 2 + rgl;
      const int srow = rgl * 32 + h32;                        // row inside the staging area, 256 B per row (128 fp16)
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          typedef _Float16 h4 __attribute__((ext_vector_type(4)));
          h4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = (_Float16)(acc[db][rg][q4 * 4 + e] * inv4[rg]);
          const int g8 = db * 8 + q4 * 2 + half;              // 8-byte granule index in the row (32 per row)
          *(h4*)(stage + srow * 256 + ((g8 ^ (srow & 31)) << 3)) = v;
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // read back: a half-wave reads one row (32 lanes x 8 B = 256 B), 2 rows per instruction, 32 instructions
#pragma unroll 4
    for (int it = 0; it < 32; it++) {
      const int srow = it * 2 + half;
      const u32x2 v = *(const u32x2*)(stage + srow * 256 + ((h32 ^ (srow & 31)) << 3));
      const int rg = round * 2 + (srow >> 5);
      const int r_in_grp = rg * 32 + (srow & 31);
      if (grp * 128 + r_in_grp < r_max)
        *(u32x2*)(p.o_part + (part_base + r_in_grp) * kDNope + wave * 128 + h32 * 4) = v;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  }  // segments
}

}  // namespace f8v2

int launch_decode_v2_fp8(const DecodeV2Params& p, dim3 grid, hipStream_t stream) {
  const void* kernel = p.win_skip ? (const void*)f8v2::mla_decode_v2_fp8_kernel<true> : (const void*)f8v2::mla_decode_v2_fp8_kernel<false>;
  const int rc = ensure_dynamic_lds(kernel, f8v2::kV2LdsB, "mla_decode_fp8");
  if (rc != MLA_OK) return rc;
  if (p.win_skip) hipLaunchKernelGGL(f8v2::mla_decode_v2_fp8_kernel<true>, grid, dim3(256), f8v2::kV2LdsB, stream, p);
  else hipLaunchKernelGGL(f8v2::mla_decode_v2_fp8_kernel<false>, grid, dim3(256), f8v2::kV2LdsB, stream, p);
  return check_launch("mla_decode_v2_fp8_kernel");
}

}  // namespace mlahip
