// Absorbed-MLA paged decode over the fp8-e4m3 block-scaled latent cache (656-byte rows: 512 fp8 | 4 fp32 scales, one per
// 128 elements | 64 bf16 rope): split-KV kernel with eight wavefronts per workgroup (two per SIMD).
//
// The structure of mla_decode_v3_kernel (decode_v3.hip: S^T = K Q^T with 16 query rows per wave, O^T += V^T P^T with 64
// output columns per wave, fixed-reference softmax placed between the P.V MFMAs, balanced chunks, the copies issued by
// wavefronts 0..3, the query staged through LDS); what differs is how a block reaches the bf16 tile the MFMA phases read:
//   * the 512 fp8 bytes and the 16 scale bytes of each of the block's 32 rows are copied global -> LDS as they are (two raw
//     stages of 16.5 KiB), the rope part goes straight into the rope buffers (it is bf16 already);
//   * at the top of body i all 512 threads turn raw block i+2 into bf16 (x = e4m3 * block scale, rounded to bf16:
//     "dequantise, then attend") in one of THREE 32 KiB tile buffers, in the swizzled layout of the bf16 kernel;
//   * the copies of block i+3 are issued right after, in one go (they have one body to land).
// LDS: 3 x 32 KiB tiles + 3 x 4 KiB rope + 2 x 16.5 KiB raw + 16 KiB P exchange + flags and tables = 159.4 KiB.
// The dominant-key correction of the bf16 kernel is not applied (its record would have to name a bf16 row); the fp8 cache
// has a wider error budget.  No reference counterpart: src/omni_npu/attention/backends/mla.py:791-792 passes
// antiquant_mode=0, antiquant_scale=None.
#include "decode_params.hpp"
#include <type_traits>
#include <cstdlib>

namespace mlahip {
namespace f8v3 {

constexpr int kBlk = 32;                                   // keys per block
constexpr int kNopeBufB = kBlk * 1024;                     // 32768
constexpr int kRopeBufB = kBlk * 128;                      // 4096
constexpr int kRopeOff = 3 * kNopeBufB;                    // 98304 (three tile buffers)
constexpr int kRawOff = kRopeOff + 3 * kRopeBufB;          // 110592
constexpr int kRawScaleOff = kBlk * 512;                   // inside a raw stage: 32 rows x 512 fp8 bytes, then 32 x 16 scale bytes
constexpr int kRawStageB = kRawScaleOff + kBlk * 16;       // 16896
constexpr int kPOff = kRawOff + 2 * kRawStageB;            // 144384
constexpr int kPBufB = 8192;                               // 4 row groups x 2 k-blocks x 64 lanes x 16 B
constexpr int kFlagOff = kPOff + 2 * kPBufB;               // 160768: restart flags, 2 x 8 dwords
constexpr int kLimitOff = kFlagOff + 64;                   // per row of the group: number of visible keys (read by masking blocks only)
constexpr int kSeenOff = kLimitOff + 512;                  // per row: the largest score that raised a restart flag
constexpr int kKTabOff = kSeenOff + 512;                   // per lane: LDS offsets of its K-fragment reads (latent, rope)
constexpr int kLdsB = kKTabOff + 512;
static_assert(kLdsB <= 160 * 1024, "LDS budget");
static_assert(8 * 16384 <= kPOff, "the query staging area ends in front of the P buffers");
constexpr int kFp8RowBytes = 656, kFp8ScaleOffB = 512, kFp8RopeOffB = 528;
constexpr int kCopyWaves = 4;                              // wavefronts 0..3 issue the copies (the older wavefront of each SIMD)
constexpr int kCopies = 6;                                 // per copying wavefront and block: 4 x two latent rows, 8 scale sets, 8 rope rows
constexpr int kAhead = 4;                                  // K fragments read ahead of the MFMA that consumes them (2 and 6 measured the same)
constexpr float kRestartThreshold = 100.f;                 // log2 units above a row's reference
constexpr int kSegCost = kPlanSegCost;
static_assert(kBlk == kPlanBlk, "the merge kernels recompute the chunk plan with these constants");

// XOR swizzles of the 16-byte granules of a row: linear over GF(2), so swz(a ^ b) = swz(a) ^ swz(b)
__device__ __forceinline__ int swz_nope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r1 ^ r3) << 3) | (r0 << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int swz_rope(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r0 ^ r3) << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int num_blocks(int len) { return len > 0 ? (len + kBlk - 1) / kBlk : 0; }
__device__ __forceinline__ int work_units(int len) { return len > 0 ? (len + kBlk - 1) / kBlk + kSegCost : 0; }
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
// inclusive scan over the 64 lanes with data-parallel-primitive moves (no LDS round trips): shifts inside the rows of 16,
// then lane 15 of rows 0 and 2 into rows 1 and 3, then lane 31 into the upper half
__device__ __forceinline__ int wave_incl_scan_dpp(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);
  return v;
}
typedef __attribute__((address_space(4))) const int32_t* ConstI32Ptr;   // scalar (constant-cache) loads


// kRG = groups of 32 query rows that can hold rows at all (4: any launch; 1 or 2: at most 32 / 64 query rows per request, as
// in the bf16 kernel): only the wavefronts that own rows run the S phase and the softmax, P.V covers kRG row groups, the
// copies move to wavefronts 4..7; all 512 threads still turn the raw block into its bf16 tile.
template <bool kWindow, int kRG = 4>
__global__ __launch_bounds__(512) void mla_decode_v3_fp8_kernel(const DecodeParams p) {
  static_assert(kRG == 1 || kRG == 2 || kRG == 4, "row groups");
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // 0..7
  const int l16 = lane & 15;                                  // QK: query row of the wave / key of a 16-key group
  const int g = lane >> 4;                                    // QK: 8-element group of a 32-deep contraction step
  const int h32 = lane & 31;
  const int half = lane >> 5;
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has its own L2.  Two families of workgroups
  // read the same bytes and are renumbered to sit on one XCD: the row groups of one chunk (more than 128 query rows)
  // stream the same cache rows; consecutive chunks belong to the same sequence and load the same queries, so every XCD
  // takes a contiguous eighth of the chunks.
  int chunk = blockIdx.x, grp = blockIdx.z;
  if ((gridDim.x & 7) == 0) {
    const int lin = blockIdx.x + gridDim.x * blockIdx.z;    // launch order
    const int j = lin >> 3;                                  // j-th workgroup of XCD lin & 7
    grp = j % gridDim.z;
    chunk = (lin & 7) * (gridDim.x >> 3) + j / gridDim.z;
  }
  const int r_max = p.max_q_len * p.num_heads;
  constexpr int kGrpRows = 32 * kRG;                          // query rows of one workgroup (blockIdx.z counts such groups)
  if (grp * kGrpRows >= r_max) return;
  const uint32_t lds0 = lds_addr_of(lds);
  // Arguments that only the start and the end of a segment need are read from the argument block where they are used
  // (through a pointer the compiler cannot see through), not held in scalar registers across the block loop: the loop
  // needs most of them itself, and scalar registers that overflow are parked in vector registers, which are short here.
  typedef __attribute__((address_space(4))) const DecodeParams* KernArgPtr;
  auto cold = [] {
    KernArgPtr kp = (KernArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(kp));
    return kp;
  };

  // ---- which blocks are mine: the balanced chunk plan (see mla_chunk_reduce_kernel, which recomputes it) ----
  // Every non-empty sequence is kSegCost units of start-up followed by its 32-key blocks, the sequences end to end, and
  // that line is cut into gridDim.x chunks of equal length; a chunk that crosses a sequence boundary runs several
  // segments; the segment of sequence b in chunk c writes partial number c + b.
  // With up to 64 sequences a lane holds one sequence's length and query range: everything the plan and the first
  // segment need comes from one round of loads issued together at the start of the kernel (each dependent round trip
  // to memory costs more than a microsecond there, with cold caches).
  int seg_b;
  int64_t v_cur, v_end, v_seq;
  int first_L = -1, first_q0 = 0, first_q1 = 0;               // the first segment's sequence, if known from the plan's loads
  {
    int tot = 0;
    const bool one_pass = p.batch <= 64;
    int my_len = 0, my_q0 = 0, my_q1 = 0;
    if (one_pass) {
      if (lane < p.batch) {
        my_len = p.seq_lens[lane];
        if (p.qsl) { my_q0 = p.qsl[lane]; my_q1 = p.qsl[lane + 1]; }
      }
      tot = work_units(my_len);
    } else {
      for (int i = lane; i < p.batch; i += 64) tot += work_units(p.seq_lens[i]);
    }
    int pe1 = 0;
    if (one_pass) { pe1 = wave_incl_scan_dpp(tot); tot = __builtin_amdgcn_readlane(pe1, 63); }
    else tot = __builtin_amdgcn_readfirstlane(wave_sum_i32(tot));
    // chunk c covers units [floor(c * tot / G), floor((c + 1) * tot / G)); with G <= 65536 that is 32-bit arithmetic:
    // c * tot / G = c * (tot / G) + c * (tot % G) / G exactly (a 64-bit division is a long software routine)
    int64_t cb, ce;
    if (gridDim.x <= 65536u) {
      const uint32_t G = gridDim.x, q = (uint32_t)tot / G, r = (uint32_t)tot - q * G;
      cb = (int64_t)chunk * q + (uint32_t)chunk * r / G;
      ce = (int64_t)(chunk + 1) * q + ((uint32_t)chunk + 1u) * r / G;
    } else {
      cb = (int64_t)chunk * tot / gridDim.x;
      ce = (int64_t)(chunk + 1) * tot / gridDim.x;
    }
    if (cb == ce) return;
    int carry = 0, b0 = 0, pb0 = 0;
    if (one_pass) {
      // the running totals do not decrease from lane to lane: the sequences that end at or before the chunk's first unit
      // are the first b0 lanes, and the last of them holds the largest such total
      const bool le = lane < p.batch && pe1 <= cb;
      b0 = __builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
      pb0 = b0 > 0 ? __builtin_amdgcn_readlane(pe1, b0 - 1) : 0;
    } else {
      for (int base = 0; base < p.batch; base += 64) {
        const int i = base + lane;
        const int c = i < p.batch ? work_units(p.seq_lens[i]) : 0;
        const int pe = wave_incl_scan_i32(c, lane) + carry;
        const bool le = i < p.batch && pe <= cb;
        b0 += __builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
        pb0 = max(pb0, wave_max_i32(le ? pe : 0));
        carry = __builtin_amdgcn_readlane(pe, 63);
      }
    }
    seg_b = __builtin_amdgcn_readfirstlane(b0) - 1;
    v_seq = __builtin_amdgcn_readfirstlane(pb0);
    v_cur = cb;
    v_end = ce;
    if (one_pass && seg_b + 1 < p.batch) {
      first_L = __builtin_amdgcn_readlane(my_len, seg_b + 1);
      first_q0 = __builtin_amdgcn_readlane(my_q0, seg_b + 1);
      first_q1 = __builtin_amdgcn_readlane(my_q1, seg_b + 1);
    }
  }

  while (v_cur < v_end) {
  seg_b++;
  if (seg_b >= p.batch) break;
  const int b = seg_b;
  const bool seg_known = first_L >= 0;                        // (only in the first pass of this loop)
  const int L = seg_known ? first_L : p.seq_lens[b];
  const int known_q0 = first_q0, known_q1 = first_q1;
  first_L = -1;
  const int64_t v_b = v_seq;
  v_seq += work_units(L);
  const int64_t v_hi = v_seq < v_end ? v_seq : v_end;
  int blk_begin = (int)(v_cur - v_b) - kSegCost;
  int blk_end = (int)(v_hi - v_b) - kSegCost;
  blk_begin = blk_begin < 0 ? 0 : blk_begin;
  blk_end = blk_end < 0 ? 0 : blk_end;
  v_cur = v_hi;
  const int nb = blk_end - blk_begin;
  if (nb <= 0) continue;
  if (threadIdx.x == 0) {
    int32_t* seg_ids = cold()->seg_ids;
    if (blk_begin == 0) seg_ids[2 * b] = chunk + b;
    if (blk_end == num_blocks(L)) seg_ids[2 * b + 1] = chunk + b;
  }
  lds_barrier();                                              // the previous segment's epilogue is done with the buffers

  int q0, qlen;
  {
    KernArgPtr kp = cold();
    const int32_t* qsl = kp->qsl;
    const int mq = kp->max_q_len;
    if (qsl && seg_known) { q0 = known_q0; qlen = known_q1 - q0; }
    else if (qsl) { q0 = qsl[b]; qlen = qsl[b + 1] - q0; }
    else { q0 = b * mq; qlen = mq; }
    qlen = qlen < mq ? qlen : mq;
  }
  const int rows = qlen * p.num_heads;
  const bool has_rows = kRG == 4 || (wave * 16 < kGrpRows && grp * kGrpRows + wave * 16 < rows);

  // this lane's query row for QK / softmax; the four lanes l16 + 16*g share it
  const int rloc = wave * 16 + l16;                           // row inside the group of 128
  const int row = grp * kGrpRows + rloc;
  const bool row_ok = row < rows && rloc < kGrpRows && L > 0;
  const int t_local = row / p.num_heads;
  const int head = row - t_local * p.num_heads;
  {
    int limit = row_ok ? (L - qlen + t_local + 1) : 0;       // keys [0, limit) are visible to this row
    limit = limit < 0 ? 0 : limit;
    if (g == 0) *(int*)(lds + kLimitOff + rloc * 4) = limit;  // read back by the blocks that have to mask (the last ones)
    if (g == 0) *(float*)(lds + kSeenOff + rloc * 4) = -INFINITY;
    if constexpr (kRG < 4) {                                  // wavefronts without rows never write their restart flags
      if (threadIdx.x < 16) *(int*)(lds + kFlagOff + threadIdx.x * 4) = 0;
    }
    // the two per-lane offsets of the K-fragment reads live in LDS and are fetched at the start of every QK phase (one
    // read instead of two registers held through the P.V phase, where registers are short)
    if (wave == 0) {
      const u32x2 kr = {(uint32_t)(l16 * 1024 + (((g << 2) ^ swz_nope(l16)) << 4)),
                        (uint32_t)(kRopeOff + l16 * 128 + (((g << 1) ^ swz_rope(l16)) << 4))};
      *(u32x2*)(lds + kKTabOff + lane * 8) = kr;
    }
  }
  const int win_skip = kWindow ? p.win_skip[b] : 0;
  const int win_blk0 = kWindow ? p.win_sink / kBlk : 0;
  const int64_t part_base = (int64_t)(chunk + b) * r_max + grp * kGrpRows;   // + row index in the group

  if (grp * kGrpRows >= rows) {
    if (row < r_max && rloc < kGrpRows && g == 0) { KernArgPtr kp = cold(); kp->lse_part[part_base + rloc] = -INFINITY; kp->corr_scale[part_base + rloc] = 0.f; }
    continue;
  }

  // ---- global -> LDS copies: wavefronts 0..3 copy eight rows of the block each, six instructions ----
  // (a copy instruction holds up the wave that issues it, and the two wavefronts of a SIMD would stall at the same moments
  // if both copied: the older one copies, the younger one keeps the matrix pipe busy)
  //   4 x two rows of 512 fp8 bytes (lane i: row 2k + i/32 of the wave's eight, granule i % 32) -> raw stage, row after row
  //   1 x the eight rows' 16 scale bytes (lanes 0..7)                                           -> behind the 32 rows
  //   1 x the eight rows' 128 rope bytes (lane i: row i/8, granule i%8, swizzled by the lane)   -> rope buffer
  // Rows past the end of the sequence re-read its last row (their scores are masked; their bytes must be finite).
  const bool copier = kRG == 4 ? wave < kCopyWaves : wave >= 8 - kCopyWaves;
  const int cw = kRG == 4 ? wave : (wave & 3);                // the copying wavefront's number among the four
  // The hardware lane number behind an opaque (and volatile) statement: what is derived from it inside the loop is
  // computed inside the loop.  Left alone the compiler hoists every loop-invariant LDS address out of the block loop, a
  // dozen registers of them, and then spills them - and a scratch reload waits for every copy in flight.
  auto lane_now = [] {
    int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(ln));
    return ln;
  };
  const int swz_rw = swz_rope((cw * 8) & 15);                  // scalar
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
  // buffer of a block (tile and rope alike): (blk - blk_begin + ph) % 3 without a division (ph = blk_begin % 3 once per segment)
  const int rope_ph = blk_begin % 3;
  auto rope_buf_of = [&](int blk) -> int {
    int r = (blk - blk_begin + rope_ph);                      // counts up by one per block from a value below 3
    r -= 3 * (int)(((uint32_t)r * 43691u) >> 17);             // r / 3 for r < 98304: one multiply, no division sequence
    return r;
  };
  auto issue_block = [&](int blk) {
    if (!copier) return;
    const int last = L - 1 - blk * kBlk;                      // last valid row of the block (>= 0)
    const uint32_t raw = lds0 + kRawOff + (blk & 1) * kRawStageB;
    const uint32_t rbuf = lds0 + kRopeOff + rope_buf_of(blk) * kRopeBufB;
    const int cblk = blk + (kWindow && blk >= win_blk0 ? win_skip : 0);   // block of the cache
    const int page = cblk >> 2;
    if (blk == blk_begin) { page_cur = page; pg_cur = load_page(page); pg_nxt = load_page(page + 1); }
    else if (page != page_cur) {
      pg_cur = (kWindow && page != page_cur + 1) ? load_page(page) : pg_nxt;   // the jump from the sink to the window
      page_cur = page;
      pg_nxt = load_page(page + 1);
    }
    const char* src = (const char*)p.cache8 + pg_cur * p.c8_sp + (int64_t)(cblk & 3) * kBlk * kFp8RowBytes;
    const int ln = lane_now();
    auto row_of = [&](int r) { return r < last ? r : last; };  // (a full block: last >= 31, nothing is clamped)
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const int r = cw * 8 + 2 * k + (ln >> 5);
      dma16_sv(src, (uint32_t)(row_of(r) * kFp8RowBytes + (ln & 31) * 16), raw + (cw * 8 + 2 * k) * 512);
    }
    dma16_sv_lanes8(src, (uint32_t)(row_of(cw * 8 + (ln & 7)) * kFp8RowBytes + kFp8ScaleOffB), raw + kRawScaleOff + cw * 128);
    {
      const int t = (ln >> 3) & 7;
      const uint32_t off = (uint32_t)(((ln & 7) ^ swz_rw ^ ((t & 1) << 2) ^ (t & 2) ^ (t >> 2)) << 4);   // swz_rope(t) = (t0 << 2) | (t1 << 1) | t2
      dma16_sv(src, (uint32_t)(row_of(cw * 8 + t) * kFp8RowBytes + kFp8RopeOffB) + off, rbuf + cw * 1024);
    }
  };
  // raw block `blk` -> bf16 tile of that block, all 512 threads: thread (row r = t / 16, c = t % 16) turns the 32 e4m3 values
  // 32c .. 32c+31 of the row (inside scale block c / 4) into four 16-byte granules of the swizzled tile row
  auto dequant_block = [&](int blk) {
    const int t = wave * 64 + lane_now();
    const int r = t >> 4, c = t & 15;
    const char* raw = lds + kRawOff + (blk & 1) * kRawStageB;
    const u32x4 w0 = *(const u32x4*)(raw + r * 512 + c * 32);
    const u32x4 w1 = *(const u32x4*)(raw + r * 512 + c * 32 + 16);
    const float sc = *(const float*)(raw + kRawScaleOff + r * 16 + (c >> 2) * 4);
    char* tile = lds + rope_buf_of(blk) * kNopeBufB + r * 1024;
    const int sw = swz_nope(r & 15);
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const u32x4 w = h ? w1 : w0;
      u32x4 o[2];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x2 x0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], false);
        const f32x2 x1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[j], true);
        bf16x2 y0, y1;
        y0[0] = (__bf16)(x0[0] * sc); y0[1] = (__bf16)(x0[1] * sc);
        y1[0] = (__bf16)(x1[0] * sc); y1[1] = (__bf16)(x1[1] * sc);
        o[j >> 1][2 * (j & 1)] = __builtin_bit_cast(uint32_t, y0);
        o[j >> 1][2 * (j & 1) + 1] = __builtin_bit_cast(uint32_t, y1);
      }
      *(u32x4*)(tile + (((4 * c + 2 * h) ^ sw) << 4)) = o[0];
      *(u32x4*)(tile + (((4 * c + 2 * h + 1) ^ sw) << 4)) = o[1];
    }
  };

  // ---- prologue: the query, then the first blocks' copies ----
  // The MFMA operand layout wants, per load instruction, 16 bytes of 64 different cache lines: read straight from
  // memory the texture addresser needs 64 cycles per instruction and the query takes ten microseconds.  So every wave
  // copies its own 16 rows global -> LDS whole (one row per instruction, into the tile buffers, which are free at the
  // start of a segment) and picks its operands from there.  The copies of the first key blocks have to wait until
  // every wave has its query in registers (one barrier).
  bf16x8 qf[18];                                             // contraction steps of 32: 16 over the latent part, 2 over rope
  if (!has_rows) {
#pragma unroll
    for (int kk = 0; kk < 18; kk++) qf[kk] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (kRG < 4) {
      // small forms: the query is staged in the first 64 KiB (tiles) by wavefronts 0..3, the raw stages and rope buffers lie
      // behind them, so the copying wavefronts ask for the first two raw blocks now, beside the query's round trip
      issue_block(blk_begin);
      if (nb > 1) issue_block(blk_begin + 1);
    }
  } else {
    // Contraction step kk of the latent part covers the 16-byte granules 16*(kk%4) + 4g' + kk/4, g' = 0..3, and lane group
    // g takes granule g' = g (rope: granules 2g' + c for step c): the K-fragment read of two lanes 16 apart must not land
    // in one aligned 32-byte piece of a row, or the LDS serves the instruction at half rate (measured: 126 against 227
    // bytes per clock and CU with eight wavefronts reading).
    KernArgPtr kp = cold();
    const int ln = lane_now();
    const int nh = kp->num_heads;
    const int r0 = grp * kGrpRows + wave * 16;               // the wave's first row
    {
      // latent part: row k of the wave is one copy instruction; lane i brings granule i ^ swz(k) (the tile swizzle)
      int t = r0 / nh, h = r0 - t * nh;
      const __bf16* qn0 = kp->q_nope;
      const int64_t st = kp->qn_st, sh = kp->qn_sh;
#pragma unroll
      for (int k = 0; k < 16; k++) {
        const bool ok = r0 + k < rows && L > 0;              // rows that do not exist read row 0 of the sequence
        const __bf16* src = qn0 + (ok ? (int64_t)(q0 + t) * st + (int64_t)h * sh : (int64_t)q0 * st);
        dma16_sv(src, (uint32_t)((ln ^ swz_nope(k)) << 4), lds0 + wave * 16384 + k * 1024);
        h++;
        if (h == nh) { h = 0; t++; }
      }
    }
    {
      // rope part: eight rows of 128 bytes per instruction, no swizzle (two reads per lane, once per segment)
      const __bf16* qr0 = kp->q_rope;
      const int64_t st = kp->qr_st, sh = kp->qr_sh;
#pragma unroll
      for (int j = 0; j < 2; j++) {
        const int rw = r0 + 8 * j + (ln >> 3);
        const bool ok = rw < rows && L > 0;
        const int t = rw / nh, h = rw - t * nh;
        const __bf16* src = qr0 + (ok ? (int64_t)(q0 + t) * st + (int64_t)h * sh : (int64_t)q0 * st) + (ln & 7) * 8;
        dma16_v(src, lds0 + kPOff + wave * 2048 + j * 1024);
      }
    }
    MLA_WAIT_VMCNT(0);
    const int ql16 = ln & 15, qg = ln >> 4;
    const uint32_t qoff = (uint32_t)(wave * 16384 + ql16 * 1024 + (((qg << 2) ^ swz_nope(ql16)) << 4));
#pragma unroll
    for (int kk = 0; kk < 16; kk++) qf[kk] = *(const bf16x8*)(lds + (qoff ^ (uint32_t)((kk >> 2) << 4)) + (kk & 3) * 256);
#pragma unroll
    for (int kk = 0; kk < 2; kk++) qf[16 + kk] = *(const bf16x8*)(lds + kPOff + wave * 2048 + ql16 * 128 + (2 * qg + kk) * 16);
#pragma unroll
    for (int kk = 0; kk < 18; kk++) asm volatile("" : "+v"(qf[kk]));           // the query stays in VGPRs
  }
  lds_barrier();                                              // every wave has read its query: the staging area is free

  f32x16 acc[2][4];                                          // [32-column block of this wave's 64][row group]
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  float m_ref = -INFINITY;       // the row's softmax reference (log2 domain), the same in its four lanes
  float l_run = 0.f;             // this lane's share of the row's sum

  // ---- per-lane LDS offsets ----
  // K-fragment reads: latent part at kbase ^ ((kk>>2) << 4), offset kg*16384 + (kk&3)*256; rope part at
  // rbase ^ ((kk-16) << 4), offset kg*2048 (kbase, rbase: the table at kKTabOff)
  const int g16 = lane >> 4, j16 = lane & 15;
  const int v_row = 4 * (g16 >> 1) + (j16 >> 2);              // + 8*rd + 16*kb
  const int v_cl = 2 * (g16 & 1) + ((j16 & 3) >> 1);
  const int v_in = (j16 & 1) * 8;
  uint32_t vbase[2];                                          // [rd]: ^ (db << 6), + kb*16384, + buffer
#pragma unroll
  for (int rd = 0; rd < 2; rd++) {
    const int rr = v_row + 8 * rd;
    vbase[rd] = (uint32_t)(rr * 1024 + v_in + (((8 * wave + v_cl) ^ swz_nope(rr & 15)) << 4));
  }
  // P^T in LDS, in the order the P.V MFMAs read it: fragment (row group rg, k-block kb) is 64 lanes x 16 B, lane
  // (n = row % 32, h) holding keys 16kb + {4h..4h+3, 8+4h..8+4h+3}.  The QK lane (row l16 of wave w, group g) holds keys
  // 16kg + 4g + {0..3}: they are the first (g < 2) or second (g >= 2) 8 bytes of lane (n, h = g & 1).
  // (worked out from the hardware lane number where it is used: a register held for it through the loop was the one the
  // compiler chose to spill, and a scratch reload waits for every copy in flight)
  auto p_w_off_now = [&]() -> uint32_t {
    const int ln = lane_now(), pg = ln >> 4, pl = ln & 15;
    return (uint32_t)(kPOff + (((wave >> 1) * 2) * 64 + (pg & 1) * 32 + (wave & 1) * 16 + pl) * 16 + (pg >> 1) * 8);   // + kg*1024 + parity*8192
  };

  // S^T for block `blk`: hand-placed K-fragment reads kAhead fragments ahead of the MFMA that consumes them, explicit
  // lgkmcnt waits, MFMAs as assembly with the scores in ordinary vector registers (the accumulation file is full of
  // output accumulators).  Dependent MFMAs of one shape with identical C and D need no padding; the two accumulators
  // alternate.  The wait after the last one (MFMA result read by the vector ALU) is the s_nop pair at the end.
  auto qk_block = [&](int blk, f32x4 (&s)[2]) {
    // the six addresses the 36 reads use (the rest is immediate offsets)
    uint32_t na[4], ra[2];
    const u32x2 kr = *(const u32x2*)(lds + kKTabOff + lane_now() * 8);
    const int tb = rope_buf_of(blk);
    na[0] = lds0 + tb * kNopeBufB + kr[0];
    ra[0] = lds0 + tb * kRopeBufB + kr[1];
#pragma unroll
    for (int b4 = 1; b4 < 4; b4++) na[b4] = na[0] ^ (uint32_t)(b4 << 4);
    ra[1] = ra[0] ^ 16u;
    bf16x8 ka[kAhead];
    // fragment j: contraction step kk = j >> 1, key group kg = j & 1; each statement is wait + MFMA + the read that
    // refills the fragment register (one statement, so that nothing is scheduled or padded in between)
#define MLA_K_ADDR(j) (((j) >> 1) < 16 ? na[(j) >> 3] : ra[((j) >> 1) - 16])
#define MLA_K_OFF(j) (((j) >> 1) < 16 ? ((j) & 1) * 16384 + (((j) >> 1) & 3) * 256 : ((j) & 1) * 2048)
#pragma unroll
    for (int i = 0; i < kAhead; i++) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ka[i]) : "v"(MLA_K_ADDR(i)), "i"(MLA_K_OFF(i)));
#pragma unroll
    for (int j = 0; j < 36; j++) {
      constexpr int D = kAhead;
      const int younger = (36 - 1 - j) < (D - 1) ? (36 - 1 - j) : (D - 1);
      if (j < 2)
        asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, 0\n\tds_read_b128 %1, %3 offset:%4"
                     : "=&v"(s[j & 1]), "+v"(ka[j % D]) : "v"(qf[j >> 1]), "v"(MLA_K_ADDR(j + D)), "i"(MLA_K_OFF(j + D)), "i"(younger));
      else if (j + D < 36)
        asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tds_read_b128 %1, %3 offset:%4"
                     : "+v"(s[j & 1]), "+v"(ka[j % D]) : "v"(qf[j >> 1]), "v"(MLA_K_ADDR(j + D)), "i"(MLA_K_OFF(j + D)), "i"(younger));
      else
        asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                     : "+v"(s[j & 1]) : "v"(ka[j % D]), "v"(qf[j >> 1]), "i"(younger));
    }
#undef MLA_K_ADDR
#undef MLA_K_OFF
    asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s[0]), "+v"(s[1]));
  };

  // ---- softmax + P.V, hand-ordered ----
  // The vector ALU is the second bottleneck of this kernel: two wavefronts share one, an MFMA of one wavefront hides about
  // four ordinary vector instructions of the other, and v_exp_f32 runs at quarter rate.  So the softmax of block i+1 is
  // written as short assembly statements placed between the P.V MFMAs of block i (the compiler would otherwise gather the
  // vector work behind the MFMAs), and it is kept to the minimum: per score one FMA, one exponential, one add, half a
  // conversion, plus the lane's maximum for the restart test (key 16*(r/4) + 4g + r%4 at sc[r]).
  // Nothing here crosses lanes: the sums are per lane and are combined in the epilogue.
  struct Sm { float t, psum; uint32_t mx; uint32_t pw[4]; };   // t = scaled max score - reference (log2); pw: bf16 pairs
#define SM_EXP2(a, b)                                                                                                   \
  asm volatile("v_fma_f32 %0, %0, %2, -%3\n\tv_fma_f32 %1, %1, %2, -%3\n\tv_exp_f32 %0, %0\n\tv_exp_f32 %1, %1"          \
               : "+v"(sc[a]), "+v"(sc[b]) : "s"(p.scale_log2), "v"(m_ref))
  auto sm_head = [&](float (&sc)[8], Sm& st) {               // the lane's maximum (4 instructions)
    asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(st.mx) : "v"(sc[0]), "v"(sc[1]), "v"(sc[2]));
    asm volatile("v_max3_f32 %0, %0, %1, %2\n\tv_max3_f32 %0, %0, %3, %4\n\tv_max_f32 %0, %0, %5"
                 : "+v"(st.mx) : "v"(sc[3]), "v"(sc[4]), "v"(sc[5]), "v"(sc[6]), "v"(sc[7]));
  };
  auto sm_pm = [&](Sm& st) {
    asm volatile("v_fma_f32 %0, %1, %2, -%3" : "=v"(st.t) : "v"(st.mx), "s"(p.scale_log2), "v"(m_ref));
  };
  auto sm_sum_lo = [&](float (&sc)[8], Sm& st) {
    asm volatile("v_add_f32 %0, %2, %3\n\tv_cvt_pk_bf16_f32 %1, %2, %3" : "=&v"(st.psum), "=v"(st.pw[0]) : "v"(sc[0]), "v"(sc[1]));
    asm volatile("v_add_f32 %0, %0, %2\n\tv_cvt_pk_bf16_f32 %1, %2, %3\n\tv_add_f32 %0, %0, %3"
                 : "+v"(st.psum), "=v"(st.pw[1]) : "v"(sc[2]), "v"(sc[3]));
  };
  auto sm_sum_hi = [&](float (&sc)[8], Sm& st) {
    asm volatile("v_add_f32 %0, %0, %2\n\tv_cvt_pk_bf16_f32 %1, %2, %3\n\tv_add_f32 %0, %0, %3"
                 : "+v"(st.psum), "=v"(st.pw[2]) : "v"(sc[4]), "v"(sc[5]));
    asm volatile("v_add_f32 %0, %0, %2\n\tv_cvt_pk_bf16_f32 %1, %2, %3\n\tv_add_f32 %0, %0, %3"
                 : "+v"(st.psum), "=v"(st.pw[3]) : "v"(sc[6]), "v"(sc[7]));
  };
  // O^T += V^T P^T for block `blk` (this wave's 64 output columns, all four row groups; kPv) with the softmax of the next
  // block's scores sc riding along (kSm).  Per k-block the two V^T fragments are held while the four P^T fragments go by
  // (two registers quads, each refilled as soon as its MFMAs are issued), every fragment feeding two MFMAs.
  // (small forms: sm_on tells whether this wavefront owns rows; one call site serves both kinds of wavefront, so that the
  // accumulators stay in the same registers - a copy the compiler puts behind an MFMA it cannot see would read them early)
  auto pv_softmax = [&](int blk, auto with_pv, auto with_sm, float (&sc)[8], Sm& st, bool sm_on) {
    constexpr bool kPv = decltype(with_pv)::value, kSm = decltype(with_sm)::value;
    const uint32_t vb = lds0 + rope_buf_of(blk) * kNopeBufB;
    const uint32_t a0 = vb + vbase[0], a1 = vb + vbase[1];    // ^ 64 for the second 32 columns, + 16384 for the second k-block
    const uint32_t a0x = a0 ^ 64u, a1x = a1 ^ 64u;
    const uint32_t pa = lds0 + (blk & 1) * kPBufB + kPOff + ((uint32_t)lane_now() << 4);   // + (rg*2 + kb)*1024
    bf16x4 v0l, v0h, v1l, v1h;
    bf16x8 pr0, pr1;
#define PV_VREAD(kb)                                                                                                   \
    asm volatile("ds_read_b64_tr_b16 %0, %4 offset:%8\n\tds_read_b64_tr_b16 %1, %5 offset:%8\n\t"                          \
                 "ds_read_b64_tr_b16 %2, %6 offset:%8\n\tds_read_b64_tr_b16 %3, %7 offset:%8"                              \
                 : "=&v"(v0l), "=&v"(v0h), "=&v"(v1l), "=&v"(v1h) : "v"(a0), "v"(a1), "v"(a0x), "v"(a1x), "i"((kb) * 16384))
#define PV_PREAD(dst, rg, kb) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(pa), "i"(((rg) * 2 + (kb)) * 1024))
#define PV_MFMA2(rg, pr, cnt)                                                                                          \
    do {                                                                                                               \
      const bf16x8 va0 = __builtin_shufflevector(v0l, v0h, 0, 1, 2, 3, 4, 5, 6, 7);                                    \
      const bf16x8 va1 = __builtin_shufflevector(v1l, v1h, 0, 1, 2, 3, 4, 5, 6, 7);                                    \
      asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_f32_32x32x16_bf16 %0, %2, %4, %0\n\tv_mfma_f32_32x32x16_bf16 %1, %3, %4, %1" \
                   : "+a"(acc[0][rg]), "+a"(acc[1][rg]) : "v"(va0), "v"(va1), "v"(pr), "i"(cnt));                      \
    } while (0)
    // (small forms only, where the matrix pipe has time to spare: the block's last MFMAs have written their accumulators
    // before anything the compiler may place behind this statement reads them)
#define PV_SETTLE(rg) asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 3" : "+a"(acc[0][rg]), "+a"(acc[1][rg]))
    if constexpr (kRG == 1) {
      if constexpr (kPv) { PV_VREAD(0); PV_PREAD(pr0, 0, 0); }
      if constexpr (kSm) { if (sm_on) { sm_head(sc, st); SM_EXP2(0, 1); SM_EXP2(2, 3); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 0); PV_VREAD(1); PV_PREAD(pr0, 0, 1); }
      if constexpr (kSm) { if (sm_on) { SM_EXP2(4, 5); SM_EXP2(6, 7); sm_pm(st); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 0); PV_SETTLE(0); }
      if constexpr (kSm) { if (sm_on) { sm_sum_lo(sc, st); sm_sum_hi(sc, st); } }
    } else if constexpr (kRG == 2) {
      if constexpr (kPv) { PV_VREAD(0); PV_PREAD(pr0, 0, 0); PV_PREAD(pr1, 1, 0); }
      if constexpr (kSm) { if (sm_on) { sm_head(sc, st); SM_EXP2(0, 1); } }
      if constexpr (kPv) PV_MFMA2(0, pr0, 1);
      if constexpr (kSm) { if (sm_on) SM_EXP2(2, 3); }
      if constexpr (kPv) { PV_MFMA2(1, pr1, 0); PV_VREAD(1); PV_PREAD(pr0, 0, 1); PV_PREAD(pr1, 1, 1); }
      if constexpr (kSm) { if (sm_on) { SM_EXP2(4, 5); SM_EXP2(6, 7); sm_pm(st); } }
      if constexpr (kPv) PV_MFMA2(0, pr0, 1);
      if constexpr (kSm) { if (sm_on) sm_sum_lo(sc, st); }
      if constexpr (kPv) { PV_MFMA2(1, pr1, 0); PV_SETTLE(0); PV_SETTLE(1); }
      if constexpr (kSm) { if (sm_on) sm_sum_hi(sc, st); }
    } else {
    (void)sm_on;
    if constexpr (kPv) { PV_VREAD(0); PV_PREAD(pr0, 0, 0); PV_PREAD(pr1, 1, 0); }
    if constexpr (kSm) sm_head(sc, st);
    if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_PREAD(pr0, 2, 0); }
    if constexpr (kSm) SM_EXP2(0, 1);
    if constexpr (kPv) { PV_MFMA2(1, pr1, 1); PV_PREAD(pr1, 3, 0); }
    if constexpr (kSm) SM_EXP2(2, 3);
    if constexpr (kPv) { PV_MFMA2(2, pr0, 1); PV_PREAD(pr0, 0, 1); }
    if constexpr (kSm) SM_EXP2(4, 5);
    if constexpr (kPv) { PV_MFMA2(3, pr1, 1); PV_VREAD(1); PV_PREAD(pr1, 1, 1); }
    if constexpr (kSm) { SM_EXP2(6, 7); sm_pm(st); }
    if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_PREAD(pr0, 2, 1); }
    if constexpr (kSm) sm_sum_lo(sc, st);
    if constexpr (kPv) { PV_MFMA2(1, pr1, 1); PV_PREAD(pr1, 3, 1); }
    if constexpr (kSm) sm_sum_hi(sc, st);
    if constexpr (kPv) { PV_MFMA2(2, pr0, 1); PV_MFMA2(3, pr1, 0); }
    }
#undef PV_SETTLE
#undef PV_VREAD
#undef PV_PREAD
#undef PV_MFMA2
  };
  // After the softmax: the last blocks of a sequence hold keys that some rows must not see (causal multi-token queries,
  // rows past the end of the sequence); only those blocks pay for the masking.  Then P^T and the restart flag go to LDS.
  auto softmax_finish = [&](int blk, float (&sc)[8], Sm& st) {
    bool front = false;
    if constexpr (kWindow) front = blk >= win_blk0 && blk * kBlk < L - p.win_size;
    if ((blk + 1) * kBlk > L - p.max_q_len + 1 || front) {
      int blk_s = blk;
      asm volatile("" : "+s"(blk_s));
      const int limit = *(const int*)(lds + kLimitOff + (wave * 16 + (lane_now() & 15)) * 4);
      const int rel = limit - blk_s * kBlk - ((lane_now() >> 4) << 2);   // score r is visible iff 16*(r/4) + r%4 < rel
      const int rel_lo = (kWindow && blk >= win_blk0) ? rel - p.win_size : -64;
      st.psum = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const int kpos = 16 * (r >> 2) + (r & 3);
        const float v = (kpos < rel && kpos >= rel_lo) ? sc[r] : 0.f;
        sc[r] = v;
        st.psum += v;
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const bf16x2 pr2 = {(__bf16)sc[2 * j], (__bf16)sc[2 * j + 1]};
        st.pw[j] = __builtin_bit_cast(uint32_t, pr2);
      }
    }
    l_run += st.psum;
    const uint32_t pw = lds0 + (blk & 1) * kPBufB + p_w_off_now();
    const u32x2 w0 = {st.pw[0], st.pw[1]}, w1 = {st.pw[2], st.pw[3]};
    asm volatile("ds_write_b64 %0, %1\n\tds_write_b64 %0, %2 offset:1024" :: "v"(pw), "v"(w0), "v"(w1) : "memory");
    const bool flag = st.t > kRestartThreshold;               // asks the workgroup to restart with better references
    const bool any = __builtin_amdgcn_ballot_w64(flag) != 0;
    if (any) {
      // (rare) the scores that outgrew the reference are remembered, per row: they become the references of the restart
      float v = flag ? st.t + m_ref : -INFINITY;
      v = fmaxf(v, __shfl_xor(v, 16, 64));
      v = fmaxf(v, __shfl_xor(v, 32, 64));
      float* seen = (float*)(lds + kSeenOff + (wave * 16 + (lane_now() & 15)) * 4);
      if (lane_now() < 16) *seen = fmaxf(*seen, v);
    }
    if (lane_now() == 0) *(int*)(lds + kFlagOff + (blk & 1) * 32 + wave * 4) = any ? 1 : 0;
  };
  // every wave reads the same eight flags: a uniform decision
  auto flags_read = [&](int blk) -> int { return *(const int*)(lds + kFlagOff + (blk & 1) * 32 + (lane_now() & 7) * 4); };
  auto flags_ask_restart = [&](int fl) -> bool { return __builtin_amdgcn_ballot_w64(fl != 0) != 0; };
  auto unpack_scores = [&](const f32x4 (&s)[2], float (&sc)[8]) {
#pragma unroll
    for (int r = 0; r < 8; r++) sc[r] = s[r >> 2][r & 3];
  };

  if constexpr (kRG < 4) {
    // a wavefront without rows publishes no probabilities: its slots of both P buffers hold zeros for the whole segment
    if (!has_rows) {
      const u32x2 z = {0u, 0u};
      const uint32_t pw = lds0 + p_w_off_now();
      asm volatile("ds_write_b64 %0, %1\n\tds_write_b64 %0, %1 offset:1024\n\tds_write_b64 %0, %1 offset:8192\n\tds_write_b64 %0, %1 offset:9216"
                   :: "v"(pw), "v"(z) : "memory");
    }
  }
  bool restart = false;
  bool early_issued = kRG < 4;   // (small forms: the first two raw blocks were requested beside the query)
  int restarts_left = 4;         // every restart raises a reference by more than 2^100: fp32 has room for three
  do {
    if (restart) {
      // a row outgrew its reference: drain, take the maxima seen so far as references, clear the sums, start over
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      const float ms = *(const float*)(lds + kSeenOff + (wave * 16 + (lane_now() & 15)) * 4);
      m_ref = fmaxf(m_ref, ms);
      l_run = 0.f;
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
      restart = false;
    }
    // ---- start-up: the first two raw blocks, dequantised into their tiles; then the third goes out ----
    if (!early_issued) {
      issue_block(blk_begin);                                 // raw stage of its parity, rope buffer 0
      if (nb > 1) issue_block(blk_begin + 1);
    }
    early_issued = false;
    MLA_WAIT_VMCNT(0);
    lds_barrier();                                            // both raw blocks have landed
    dequant_block(blk_begin);
    if (nb > 1) dequant_block(blk_begin + 1);
    lds_barrier();                                            // tiles complete, both raw stages free
    if (nb > 2) issue_block(blk_begin + 2);
    // ---- block 0: QK, softmax, publish ----
    {
      f32x4 s[2];
      Sm st;
      if (has_rows) {
      qk_block(blk_begin, s);
      if (m_ref == -INFINITY) {
        // the first block fixes the reference: the row's largest score over all 32 keys (visible or not: any finite
        // reference within 2^100 of the true maximum is as good as another), the same value in the row's four lanes
        float mx = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                         fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        m_ref = mx * p.scale_log2;
      }
      float sc[8];
      unpack_scores(s, sc);
      pv_softmax(blk_begin, std::false_type{}, std::true_type{}, sc, st, true);
      softmax_finish(blk_begin, sc, st);
      }
    }
    // Everything the loop keeps in registers is touched here: a value that was parked in scratch during the prologue is
    // brought back (and waited for) now, not at its first use inside the loop.
    asm volatile("" :: "v"(vbase[0]), "v"(vbase[1]), "v"(m_ref), "v"(l_run));
    // ---- steady state: dequantise block i+2, request block i+3, QK(i+1), then P.V(i) with the softmax of block i+1 ----
    for (int i = 0; i + 1 < nb; i++) {
      const int blk = blk_begin + i;
      // tile i+1 is complete, raw block i+2 has landed (after this wait and the barrier), P(i) is published, everyone is
      // done with P.V(i-1), i.e. with tile (i+2) % 3, and with raw stage (i+1) & 1
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      const int fl = flags_read(blk);
      // The copying wavefronts dequantise their half of block i+2 (rows 0..15) now, the others theirs (rows 16..31) at the
      // end of the body: the two wavefronts of a SIMD then run half a phase apart, and one's conversions and LDS writes
      // sit under the other's MFMAs.  Both halves are done before the next barrier, which is when the tile is read.
      // (measured on batch 256 x 2 tokens, 16k-32k keys: all wavefronts at the top 3840 us; this order 3663; the others
      // between their S and P.V phases 3725; the two roles swapped 3974)
      if (copier && i + 2 < nb) dequant_block(blk + 2);
      if (i + 3 < nb) issue_block(blk + 3);
      f32x4 s[2];
      if (has_rows) qk_block(blk + 1, s);
      if (restarts_left > 0 && flags_ask_restart(fl)) { restart = true; restarts_left--; break; }
      Sm st;
      float sc[8];
      unpack_scores(s, sc);
      pv_softmax(blk, std::true_type{}, std::true_type{}, sc, st, has_rows);
      if (has_rows) softmax_finish(blk + 1, sc, st);
      if (!copier && i + 2 < nb) dequant_block(blk + 2);
    }
    if (!restart) {
      const int blk = blk_end - 1;
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      if (restarts_left > 0 && flags_ask_restart(flags_read(blk))) { restart = true; restarts_left--; }
      else { float sc[8]; Sm st; pv_softmax(blk, std::true_type{}, std::false_type{}, sc, st, true); }
    }
  } while (restart);

  // ---- epilogue ----
  // (lane-derived values are worked out again from the hardware lane number: nothing of them has to live through the loop)
  lds_barrier();                                              // all PV done; tile buffers and P buffers are free
  const int e_ln = lane_now();
  const int e_l16 = e_ln & 15, e_g = e_ln >> 4, e_h32 = e_ln & 31, e_half = e_ln >> 5;
  const int e_rloc = wave * 16 + e_l16;
  {
    const int e_row = grp * kGrpRows + e_rloc;
    // the row's four lanes combine their sums
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const float corr = 0.f;                                   // no dominant-key correction over the fp8 cache
    const __bf16* vrow = nullptr;
    KernArgPtr kp = cold();
    if (e_g == 0) {
      *(float*)(lds + kPOff + (e_rloc & 31) * 16 + (e_rloc >> 5) * 4) = inv;
      if (e_row < r_max && e_rloc < kGrpRows) {
        const int64_t pr = part_base + e_rloc;
        kp->lse_part[pr] = l_tot > 0.f ? (m_ref + fast_log2(l_tot)) * kLn2 : -INFINITY;
        kp->corr_scale[pr] = corr;
        kp->corr_row[pr] = vrow;
      }
    }
  }
  lds_barrier();
  const f32x4 inv4 = *(const f32x4*)(lds + kPOff + e_h32 * 16);
  // transpose through this wave's private 16 KiB: 128 rows x 64 columns, fp16 (128 bytes per row, 8-byte slots XORed
  // with the row so that neither the writes nor the reads collide)
  char* stage = lds + wave * 16384;
  _Float16* o_part_c = cold()->o_part;
#pragma unroll
  for (int rg = 0; rg < kRG; rg++) {
    const int srow = rg * 32 + e_h32;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
      for (int q4 = 0; q4 < 4; q4++) {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        h4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) v[e] = (_Float16)(acc[db][rg][q4 * 4 + e] * inv4[rg]);
        const int g8 = db * 8 + q4 * 2 + e_half;              // 8-byte slot in the row (16 per row)
        *(h4*)(stage + srow * 128 + ((g8 ^ ((srow >> 1) & 15)) << 3)) = v;
      }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  // read back: 16 lanes read one row (128 B), four rows per instruction
#pragma unroll 4
  for (int it = 0; it < 8 * kRG; it++) {
    const int srow = it * 4 + e_g;
    const u32x2 v = *(const u32x2*)(stage + srow * 128 + ((e_l16 ^ ((srow >> 1) & 15)) << 3));
    if (grp * kGrpRows + srow < r_max)
      *(u32x2*)(o_part_c + (part_base + srow) * kDNope + wave * 64 + e_l16 * 4) = v;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }  // segments
}

}  // namespace f8v3

template <bool kWindow, int kRG>
static int launch_form_fp8(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  const int rc = ensure_dynamic_lds((const void*)f8v3::mla_decode_v3_fp8_kernel<kWindow, kRG>, f8v3::kLdsB, "mla_decode_v3_fp8_kernel");
  if (rc != MLA_OK) return rc;
  hipLaunchKernelGGL((f8v3::mla_decode_v3_fp8_kernel<kWindow, kRG>), grid, dim3(512), f8v3::kLdsB, stream, p);
  return check_launch("mla_decode_v3_fp8_kernel");
}
template <bool kWindow>
static int launch_rows_fp8(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  // requests with at most 32 / 64 query rows (tokens x heads) take the forms that leave the missing rows out
  const int64_t r_max = (int64_t)p.max_q_len * p.num_heads;
  // (all three forms get their LDS limit with the family's first launch: a later launch under stream capture finds them ready)
  {
    int rc = ensure_dynamic_lds((const void*)f8v3::mla_decode_v3_fp8_kernel<kWindow, 1>, f8v3::kLdsB, "mla_decode_v3_fp8_kernel");
    if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)f8v3::mla_decode_v3_fp8_kernel<kWindow, 2>, f8v3::kLdsB, "mla_decode_v3_fp8_kernel");
    if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)f8v3::mla_decode_v3_fp8_kernel<kWindow, 4>, f8v3::kLdsB, "mla_decode_v3_fp8_kernel");
    if (rc != MLA_OK) return rc;
  }
  if (r_max <= 32) return launch_form_fp8<kWindow, 1>(p, grid, stream);
  if (r_max <= 64) return launch_form_fp8<kWindow, 2>(p, grid, stream);
  // (few chunks: the rows are cut into groups of 32 or 64 with a workgroup each, as in the kernel over the bf16 cache)
  {
    const int64_t wgs = (int64_t)grid.x * grid.z;
    if (wgs * 4 <= 256) { grid.z = (unsigned)((r_max + 31) / 32); return launch_form_fp8<kWindow, 1>(p, grid, stream); }
    if (wgs * 2 <= 256) { grid.z = (unsigned)((r_max + 63) / 64); return launch_form_fp8<kWindow, 2>(p, grid, stream); }
  }
  return launch_form_fp8<kWindow, 4>(p, grid, stream);
}

int launch_decode_v3_fp8(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  if (p.win_skip) return launch_rows_fp8<true>(p, grid, stream);
  return launch_rows_fp8<false>(p, grid, stream);
}

}  // namespace mlahip
