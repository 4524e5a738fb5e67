// Absorbed-MLA paged decode, second-generation kernel for the bf16 cache (dense and row-list sources).
//
// Same contract as mla_decode_bf16_kernel in decode.hip (reference call:
// src/omni_npu/attention/backends/mla.py:781-804); what changed is how a workgroup spends its LDS and MFMA issue slots.
//
// A wavefront can issue one LDS instruction per ~17 clocks, and a transposed read delivers only 8 bytes per lane, so
// "every wave reads all of V^T for its own 32 rows" (two transposed reads per MFMA) makes the P.V phase LDS-issue bound.
// Here the two products are partitioned differently:
//   S^T = K Q^T      wave w owns query rows 32w..32w+31 (its 576-wide query stays in registers), all 32 tokens of a block;
//   O^T += V^T P^T   wave w owns output columns d in [128w, 128w+128) for ALL 128 rows: a V^T fragment is read once and
//                    feeds four MFMAs (one per row group), and the four P^T blocks (2 KiB each, bf16) plus a restart
//                    flag per row travel through LDS once per block.
// Per 32 tokens a wave issues 36 + 16 + 8 + ~4 LDS instructions instead of 100, for the same 68 MFMAs.
//
// Pipeline (one barrier per 32-token block):  body i = [barrier] QK(i+1) | PV(i) overlapped with softmax(i+1) | publish P(i+1).
// Blocks live in 4 nope buffers (32 KiB) and 3 rope buffers (4 KiB); the copies of block i+3 are spread over the QK phase of
// body i, so two blocks are always in flight.
//
// No accumulator rescaling in the steady state.  The 256 output accumulators live in the accumulation register file, which
// vector ALU instructions cannot touch, so the usual online-softmax rescale would cost three instructions per element.
// Instead every row fixes its reference m_ref at the largest score of its first block and uses
// P = exp2(s - m_ref) from then on: bf16 and fp32 share one exponent range, so P may grow to 2^100 without loss of
// relative precision.  If a later score exceeds m_ref by more than 100 (log2 units; e^69 in weight) the row raises a flag
// that travels with P, and the whole workgroup restarts its segment with the row maxima seen so far as references.  Each
// restart raises a reference by more than 100, so at most a few can happen; realistic logits never trigger one.
// Partials are written as fp16 (normalised values, |o| <= max|V|) through an LDS transpose so that global stores are row
// contiguous; log-sum-exps as fp32.  With a fixed reference a row's most probable key no longer has probability exactly 1,
// so its bf16 rounding error is recorded beside the partial and taken out again by mla_chunk_reduce_kernel.
#include "decode_v2_params.hpp"
#include <type_traits>
#include <cstdlib>

namespace mlahip {

#ifndef MLA_V2_QK_AHEAD
#define MLA_V2_QK_AHEAD 6
#endif
#ifndef MLA_V2_PV_AHEAD
#define MLA_V2_PV_AHEAD 2
#endif
constexpr int kQkAheadV2 = MLA_V2_QK_AHEAD, kPvAheadV2 = MLA_V2_PV_AHEAD;   // LDS read-ahead depth, in fragments
constexpr int kBlk = 32;                                   // tokens per block
constexpr int kV2NopeBufB = kBlk * 1024;                   // 32768
constexpr int kV2RopeBufB = kBlk * 128;                    // 4096
constexpr int kV2RopeOff = 4 * kV2NopeBufB;                // 131072
constexpr int kV2POff = kV2RopeOff + 3 * kV2RopeBufB;      // 143360
constexpr int kV2PBufB = 8192;                             // 4 row groups x 2 k-blocks x 64 lanes x 16 B
constexpr int kV2AOff = kV2POff + 2 * kV2PBufB;            // 159744: rescale factors, 2 x 512 B
constexpr int kV2LdsB = kV2AOff + 2 * 512;                 // 160768
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

// kWindow (dense only): static sink keys followed by a sliding window.  The kernel walks a shortened sequence: the
// blocks between the sink and the first block of the window are left out of the block numbering (block v >= sink blocks
// is block v + skip of the cache), so the chunk plan, the ring buffers and the end-of-sequence masking work on the
// shortened length unchanged; what differs is the address of a block and one more mask at the window's front.
template <bool kSparse, bool kWindow>
__global__ __launch_bounds__(256, 1) void mla_decode_v2_kernel(const DecodeV2Params p) {
  static_assert(!(kSparse && kWindow), "the window variant reads the paged cache");
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h32 = lane & 31;
  const int half = lane >> 5;
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has its own L2.  Two families of workgroups
  // read the same bytes and are renumbered to sit on one XCD: the row groups of one chunk (more than 128 query rows:
  // several tokens per sequence) stream the same cache rows, next to each other in the XCD's queue so that they run at
  // the same time; and consecutive chunks belong to the same sequence and load the same queries, so every XCD takes a
  // contiguous eighth of the chunks (the query rows then come from memory once per sequence, not once per chunk).
  int chunk = blockIdx.x, grp = blockIdx.z;
  if ((gridDim.x & 7) == 0) {
    const int lin = blockIdx.x + gridDim.x * blockIdx.z;    // launch order
    const int j = lin >> 3;                                  // j-th workgroup of XCD lin & 7
    grp = j % gridDim.z;
    chunk = (lin & 7) * (gridDim.x >> 3) + j / gridDim.z;
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
  // window variant: blocks left out behind the sink, and the first block that is not a sink block
  const int win_skip = kWindow ? p.win_skip[b] : 0;
  const int win_blk0 = kWindow ? p.win_sink / kBlk : 0;
  const int64_t part_base = (int64_t)(chunk + b) * r_max + grp * 128;   // + row index in the group

  if (grp * 128 >= rows) {
    if (row < r_max && half == 0) { p.lse_part[part_base + wave * 32 + h32] = -INFINITY; p.corr_scale[part_base + wave * 32 + h32] = 0.f; }
    continue;
  }

  // ---- global -> LDS copies: 9 per lane and block (8 nope rows of 1 KiB per wave, one rope instruction of 8 rows) ----
  // Row r of a block goes to nope buffer row r (granule g at position g ^ swz(r)) and rope buffer row r.  All addresses
  // are a scalar base plus a per-lane 32-bit offset that does not change from block to block.
  uint32_t dma_off[4];
#pragma unroll
  for (int j = 0; j < 4; j++) dma_off[j] = (uint32_t)((lane ^ v2_swz_nope((wave * 4 + j) & 15)) << 4);
  const uint32_t rope_off = (uint32_t)(((lane & 7) ^ v2_swz_rope((wave * 8 + (lane >> 3)) & 15)) << 4);
  const uint32_t n_sr2 = (uint32_t)p.nope_sr * 2u, r_sr2 = (uint32_t)p.rope_sr * 2u;       // row strides in bytes
  const uint32_t rope_voff = (uint32_t)(lane >> 3) * r_sr2 + rope_off;                      // full blocks: row 8*wave + lane/8

  // dense source: the page of the block being copied and the next one are kept in scalar registers, so the block-table
  // load is never waited for in the loop
  ConstI32Ptr bt = (ConstI32Ptr)(p.block_table) + (kSparse ? 0 : (int64_t)b * p.bt_stride);
  ConstI32Ptr srows = (ConstI32Ptr)(p.sparse_rows) + (kSparse ? (int64_t)b * p.sparse_stride : 0);
  const int64_t max_row = p.num_pages * p.page_size - 1;
  // Row list (kSparse): the 32 cache rows of the block whose copies go out next travel in one vector register, lane r
  // holding the row of key r, and every copy picks its row with v_readlane.  (A scalar load per copy would need a full
  // lgkmcnt wait in front of every copy, and that wait also drains the K-fragment reads of the QK phase in flight: nine
  // drains per block.)  The load for block X+1 is issued in front of the copies of block X, so the wait that lets a
  // block's copies land also covers it (vector memory returns in order).
  uint32_t ids_cur = 0, ids_nxt = 0;
  auto ids_load = [&](int blk_x) {
    if constexpr (kSparse) {
      int tok = blk_x * kBlk + (lane & 31);
      tok = tok < L ? tok : L - 1;
      tok = tok < 0 ? 0 : tok;
      const int32_t* src = p.sparse_rows + (int64_t)b * p.sparse_stride + tok;
      asm volatile("global_load_dword %0, %1, off" : "=v"(ids_nxt) : "v"(src) : "memory");
    }
  };
  // after a wait that covers the load: the register is complete, hand it to the copies of the coming block
  auto ids_rotate = [&] {
    if constexpr (kSparse) {
      asm volatile("" : "+v"(ids_nxt));
      ids_cur = ids_nxt;
    }
  };
  auto load_page = [&](int page) -> int64_t {
    page = page < p.max_blocks ? page : p.max_blocks - 1;
    int64_t pg = bt[page];
    return pg < 0 ? 0 : (pg >= p.num_pages ? p.num_pages - 1 : pg);
  };
  int page_cur = 0;
  int64_t pg_cur = 0, pg_nxt = 0;
  auto issue_reset = [&]() {
    if constexpr (!kSparse) {
      page_cur = (blk_begin + (kWindow && blk_begin >= win_blk0 ? win_skip : 0)) >> 2;
      pg_cur = load_page(page_cur);
      pg_nxt = load_page(page_cur + 1);
    }
  };
  // The nine copies of a block are issued one at a time ("pieces" 0..8) so that they can be spread over the MFMAs of the
  // QK phase: piece k copies nope rows 4*wave + k/2 (+16 for odd k) for k < 8, piece 8 the wave's eight rope rows.  Rows
  // past the end of the sequence re-read its last row (their scores are masked).
  struct IssueCtx { const char* np; const char* rp; const char* a0; const char* a1; uint32_t nbuf, rbuf; int last, tok0; };
  auto issue_begin = [&](int blk) -> IssueCtx {
    IssueCtx c;
    c.tok0 = blk * kBlk;
    c.last = L - 1 - c.tok0;                                  // last valid row of the block (>= 0)
    c.nbuf = lds0 + (blk & 3) * kV2NopeBufB;
    c.rbuf = lds0 + kV2RopeOff + (blk % 3) * kV2RopeBufB;
    if constexpr (kSparse) {
      c.np = (const char*)p.nope;
      c.rp = (const char*)p.rope;
    } else {
      const int cblk = blk + (kWindow && blk >= win_blk0 ? win_skip : 0);   // block of the cache
      const int page = cblk >> 2;
      if (page != page_cur) {
        // the next page's number is only asked for here (raw: clamping it now would wait for the load); it is clamped
        // when it becomes the current page, four blocks later
        if (kWindow && page != page_cur + 1) pg_cur = load_page(page);         // the jump from the sink to the window
        else pg_cur = pg_nxt < 0 ? 0 : (pg_nxt >= p.num_pages ? p.num_pages - 1 : pg_nxt);
        page_cur = page;
        const int pn = page + 1 < p.max_blocks ? page + 1 : p.max_blocks - 1;
        pg_nxt = bt[pn];
      }
      const uint32_t row0 = (uint32_t)(cblk & 3) * kBlk;
      c.np = (const char*)p.nope + pg_cur * p.nope_sp * 2 + (uint64_t)row0 * n_sr2;
      c.rp = (const char*)p.rope + pg_cur * p.rope_sp * 2 + (uint64_t)row0 * r_sr2;
    }
    c.a0 = c.np + (uint64_t)(wave * 4) * n_sr2;               // full dense blocks: running row addresses
    c.a1 = c.a0 + (uint64_t)n_sr2 * 16;
    return c;
  };
  // kFull: every row of the block exists and the source is the paged cache: plain pointer increments
  // kVecIds (row list only): the rows come from ids_cur instead of scalar loads
  auto issue_piece = [&](IssueCtx& c, int k, auto full, auto vec_ids) {
    constexpr bool kFull = decltype(full)::value && !kSparse;
    constexpr bool kVecIds = decltype(vec_ids)::value && kSparse;
    auto clampi = [&](int64_t s_) -> int64_t { return s_ < 0 ? 0 : (s_ > max_row ? max_row : s_); };
    auto row_of = [&](int re) -> int32_t {
      if constexpr (kVecIds) return (int32_t)__builtin_amdgcn_readlane((int)ids_cur, re);
      else return srows[c.tok0 + re];
    };
    if (k < 8) {
      const int j = k >> 1;
      const int r = (k & 1) * 16 + wave * 4 + j;
      if constexpr (kFull) {
        if ((k & 1) == 0) dma16_sv(c.a0, dma_off[j], c.nbuf + r * 1024);
        else { dma16_sv(c.a1, dma_off[j], c.nbuf + r * 1024); c.a0 += n_sr2; c.a1 += n_sr2; }
      } else {
        const int re = r < c.last ? r : c.last;
        if constexpr (kSparse) dma16_sv(c.np + clampi(row_of(re)) * n_sr2, dma_off[j], c.nbuf + r * 1024);
        else dma16_sv(c.np + (uint64_t)re * n_sr2, dma_off[j], c.nbuf + r * 1024);
      }
    } else {
      if constexpr (kSparse) {
        int32_t mine = 0;                                     // lane's row = 8*wave + lane/8, picked from 8 uniform values
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const int r = wave * 8 + j;
          const int32_t sj = row_of(r < c.last ? r : c.last);
          mine = (lane >> 3) == j ? sj : mine;
        }
        dma16_v(c.rp + clampi(mine) * r_sr2 + rope_off, c.rbuf + wave * 1024);
      } else if constexpr (kFull) {
        dma16_sv(c.rp + (uint64_t)(wave * 8) * r_sr2, rope_voff, c.rbuf + wave * 1024);
      } else {
        const int r = wave * 8 + (lane >> 3);
        const int re = r < c.last ? r : c.last;
        dma16_sv(c.rp, (uint32_t)re * r_sr2 + rope_off, c.rbuf + wave * 1024);
      }
    }
  };
  auto issue_block = [&](int blk) {
    IssueCtx c = issue_begin(blk);
#pragma unroll
    for (int k = 0; k < 9; k++) issue_piece(c, k, std::false_type{}, std::integral_constant<bool, kSparse>{});
  };
  // Row list: the rows of the first kLead blocks are fetched together (one round trip) before any copy goes out
  uint32_t ids_head[kLead] = {};
  auto issue_first = [&]() {
    issue_reset();
    if constexpr (kSparse) {
#pragma unroll
      for (int j = 0; j < kLead; j++) {
        int tok = (blk_begin + j) * kBlk + (lane & 31);
        tok = tok < L ? tok : L - 1;
        tok = tok < 0 ? 0 : tok;
        const int32_t* src = p.sparse_rows + (int64_t)b * p.sparse_stride + tok;
        asm volatile("global_load_dword %0, %1, off" : "=v"(ids_head[j]) : "v"(src) : "memory");
      }
      if constexpr (kLead == 3)
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(ids_head[0]), "+v"(ids_head[1]), "+v"(ids_head[2])::"memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" : "+v"(ids_head[0]), "+v"(ids_head[1])::"memory");
      ids_cur = ids_head[0];
    }
    issue_block(blk_begin);
  };
  auto issue_next_two = [&]() {
    if constexpr (kSparse) {
#pragma unroll
      for (int j = 1; j < kLead; j++)
        if (j < nb) {
          ids_cur = ids_head[j];
          issue_block(blk_begin + j);
        }
    } else {
#pragma unroll 1
      for (int j = 1; j < kLead && j < nb; j++) issue_block(blk_begin + j);
    }
  };

  // ---- prologue: the first block's copies go out, then the query loads; both are waited for together ----
  issue_first();
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
  float top_p = 0.f;             // largest probability (relative to m_ref) among the visible keys so far ...
  int top_tok = -1;              // ... and the position of that key in the sequence's key list

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
    const uint32_t nb32 = lds0 + (blk & 3) * kV2NopeBufB + kbase;     // buffers are 4 KiB aligned: the XORs below stay exact
    const uint32_t rb32 = lds0 + (blk % 3) * kV2RopeBufB + rbase;
    IssueCtx ic;
    if constexpr (kIssue) { ids_load(blk_issue + 1); ic = issue_begin(blk_issue); }
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
      if constexpr (kIssue) if ((kk & 3) == 1) issue_piece(ic, kk >> 2, std::integral_constant<bool, kIssueMode == 2>{}, std::true_type{});
      if (kk == 27) mid_hook();
    }
#undef MLA_K_READ
    asm volatile("s_nop 7\n\ts_nop 7" : "+v"(s));
  };

  // Softmax of block `blk` from raw scores s, cut into eight straight-line steps so that it can be interleaved with the
  // P.V MFMAs of the previous block (step k is called after the k-th group of four MFMAs; the MFMAs run 32 clocks each
  // while the vector ALU is otherwise idle).  The row maximum is taken over all 32 scores of the block, visible or not:
  // it only serves as a reference, and any finite reference within 2^100 of the true maximum is as good as another.
  // Which of the row's 32 probabilities is the largest: the element number travels in the five low mantissa bits of the
  // (positive) values through an unsigned maximum, so no compare-and-select chain and no branch is needed.  Two values
  // closer than 2^-18 relative may swap places, which only matters to a correction that is itself a rounding error.
  auto argmax_pack = [&](const f32x16& s) -> uint32_t {
    // The tagging is left to the compiler on purpose: the probabilities come out of v_exp_f32, and a vector-ALU
    // instruction that reads the result of a transcendental one needs a wait state in between, which the compiler only
    // inserts in front of instructions it can see into (not in front of inline assembly).  The maximum chain is plain
    // assembly without side effects (the optimiser mangles the equivalent C++ reduction); it only reads tagged values.
    uint32_t u[16];
#pragma unroll
    for (int r = 0; r < 16; r++) u[r] = (__float_as_uint(s[r]) & ~31u) | (uint32_t)r;
    uint32_t pk = u[0];
#pragma unroll
    for (int r = 1; r < 15; r += 2) asm("v_max3_u32 %0, %1, %2, %3" : "=v"(pk) : "v"(pk), "v"(u[r]), "v"(u[r + 1]));
    asm("v_max_u32 %0, %1, %2" : "=v"(pk) : "v"(pk), "v"(u[15]));
    pk |= (uint32_t)(lane_now() >> 1) & 16u;                 // bit 4: upper half of the wavefront
    const auto sw = __builtin_amdgcn_permlane32_swap(pk, pk, false, false);
    return max((uint32_t)sw[0], (uint32_t)sw[1]);
  };
  struct SoftmaxState { float neg_ref, flag, pm; uint32_t pk; bf16x8 pb[2]; float psum; };
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
      st.pm = fast_exp2(__builtin_fmaf(mx_raw, p.scale_log2, st.neg_ref));   // bit-identical to that score's probability below
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
    } else if (step == 6) {
      st.pk = argmax_pack(s);
    }
  };
  // After the steps: the last blocks of a sequence hold keys that some rows must not see (causal multi-token queries,
  // rows past the end of the sequence); only those blocks pay for the masking.  Then P^T and the flag go to LDS.
  auto softmax_finish = [&](int blk, f32x16& s, SoftmaxState& st) {
    // window variant: the blocks right behind the sink hold keys older than some row's window (fewer than 32 + the
    // number of query tokens of them, so at most two blocks)
    bool front = false;
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
      float pv = fmaxf(s[0], s[1]);                           // largest VISIBLE probability of the row in this block
#pragma unroll
      for (int r = 2; r < 16; r += 2) pv = fmaxf(pv, fmaxf(s[r], s[r + 1]));
      st.pm = half_max(pv);
      st.pk = argmax_pack(s);
    }
    // Remember the row's most probable key: the bf16 rounding of its probability is the largest single error of the
    // P.V product when the softmax is peaked, and the merge kernel takes it out again.
    {
      const bool nw = st.pm > top_p;
      top_p = nw ? st.pm : top_p;
      const int e = (int)(st.pk & 15u);
      top_tok = nw ? blk * kBlk + (int)((st.pk >> 2) & 4u) + 8 * (e >> 2) + (e & 3) : top_tok;
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
    const uint32_t vb32 = lds0 + (blk & 3) * kV2NopeBufB;
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
    const char* vb = lds + (blk & 3) * kV2NopeBufB;
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
      top_p = 0.f;
      top_tok = -1;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
      issue_first();
      restart = false;
    }
    ids_load(blk_begin + kLead);                              // (older than the copies below: their wait covers it)
    issue_next_two();
    // ---- block 0: QK, softmax, publish ----
    {
      if (kLead > 2 && nb > 2) MLA_WAIT_VMCNT(18); else if (nb > 1) MLA_WAIT_VMCNT(9); else MLA_WAIT_VMCNT(0);
      lds_barrier();
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
                 "v"(top_p), "v"(top_tok), "v"(dma_off[0]), "v"(dma_off[1]), "v"(dma_off[2]), "v"(dma_off[3]), "v"(rope_off),
                 "v"(rope_voff));
    // ---- steady state: QK(i+1), then P.V(i) with the softmax of block i+1 riding along ----
    for (int i = 0; i + 1 < nb; i++) {
      const int blk = blk_begin + i;
      // block i+1 has landed, P(i) is published, everyone is done with P.V(i-1)
      if (kLead > 2 && i + 2 < nb) MLA_WAIT_VMCNT(9); else MLA_WAIT_VMCNT(0);
      ids_rotate();
      lds_barrier();
      const f32x4 fl = flags_read(blk);
      f32x16 s;
      PvHead head;
      auto hook = [&] { pv_head_read(blk, head); };
      if (i + kLead >= nb) qk_block(blk + 1, s, std::integral_constant<int, 0>{}, 0, hook);
      else if (kSparse || L - 1 - (blk + kLead) * kBlk < kBlk - 1) qk_block(blk + 1, s, std::integral_constant<int, 1>{}, blk + kLead, hook);
      else qk_block(blk + 1, s, std::integral_constant<int, 2>{}, blk + kLead, hook);
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
    // Rows whose most probable key carries more than 1/16 of the weight leave a note for the merge kernel: the rounding
    // error of that key's probability (already divided by l) and the address of its latent vector in the cache.
    float corr = 0.f;
    const __bf16* vrow = p.nope;
    if (row_ok && top_tok >= 0 && top_p * 16.f > l_tot) {
      corr = (top_p - (float)(__bf16)top_p) * inv;
      if constexpr (kSparse) {
        int64_t slot = p.sparse_rows[(int64_t)b * p.sparse_stride + top_tok];
        slot = slot < 0 ? 0 : (slot > max_row ? max_row : slot);
        vrow = p.nope + slot * p.nope_sr;
      } else {
        const int ctok = top_tok + ((kWindow && top_tok >= p.win_sink) ? win_skip * kBlk : 0);   // position in the cache
        int page = ctok / kPage;
        page = page < p.max_blocks ? page : p.max_blocks - 1;
        int64_t pg = p.block_table[(int64_t)b * p.bt_stride + page];
        pg = pg < 0 ? 0 : (pg >= p.num_pages ? p.num_pages - 1 : pg);
        vrow = p.nope + pg * p.nope_sp + (int64_t)(ctok % kPage) * p.nope_sr;
      }
    }
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


// N-way merge of the partials of the query rows (src/omni_npu/attention/ops.py:109-141), for the chunk layout written
// by mla_decode_v2_kernel.  The partials of sequence b are those of the chunks that hold blocks of it, numbered
// chunk + b.  A wavefront merges kRedRows consecutive rows of one sequence (lane l owns columns 8l..8l+7): it derives
// the chunk list once, fetches the per-row records of up to kRedParts partials with scalar loads, then asks for the
// partials and the latent vectors of the flagged dominant keys together before it uses any of them - the kernel is a
// chain of dependent memory round trips, and this keeps the vector part of the chain at one.  (One row per wave keeps it
// at four waves per SIMD; the gathers of the dominant keys' vectors are a third of its time.)
// With many partials per sequence (few sequences, long contexts: up to 257 partials of one row) a single wavefront would
// walk them in dozens of dependent round trips, so the kWide form gives a row to a whole workgroup: wavefront w merges
// every fourth partial, sixteen per pass, and the four running states are merged through LDS at the end.
// With one chunk per sequence (large batches) a row has one partial, or two where a chunk border falls inside its
// sequence: the kFew form then gives a wavefront four rows of two partials, a quarter of the wavefronts and rounds.
constexpr int kRedPartsNarrow = 6, kRedPartsWide = 16, kRedPartsFew = 2, kRedRowsFew = 4;
template <bool kWide, bool kFew>
__global__ __launch_bounds__(256) void mla_chunk_reduce_kernel(const ChunkReduceParams p) {
  constexpr int kRedParts = kWide ? kRedPartsWide : (kFew ? kRedPartsFew : kRedPartsNarrow);
  constexpr int kRedRows = kFew ? kRedRowsFew : 1;
  __shared__ float comb_ml[kWide ? 8 : 1];                  // wide: running maximum and sum of wavefronts 0..3
  __shared__ float comb_a[kWide ? 4 * 64 * 8 : 1];          //       and their unnormalised rows
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r_max = p.max_q_len * p.num_heads;
  const int groups = (r_max + kRedRows - 1) / kRedRows;     // row groups per sequence
  // (the wave number is made a scalar: everything derived from it, the addresses of the per-row records included, then
  // lives in scalar registers and is fetched with scalar loads)
  const int64_t gw_first = kWide ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
  const int64_t gw_step = kWide ? (int64_t)gridDim.x : (int64_t)gridDim.x * 4;
  for (int64_t gw = gw_first; gw < (int64_t)p.batch * groups; gw += gw_step) {
  const int b = (int)(gw / groups);
  const int row0 = (int)(gw - (int64_t)b * groups) * kRedRows;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  qlen = qlen < p.max_q_len ? qlen : p.max_q_len;
  const int rows = qlen * p.num_heads;
  if (row0 >= rows) continue;

  // (everything that depends on b only is requested together: one memory round trip, not three)
  const int id_first = p.seg_ids[2 * b], id_last = p.seg_ids[2 * b + 1];
  const int mine = v2_work_units(p.seq_lens[b]);
  int tot_units = 0, before = 0;
  for (int i = lane; i < p.batch; i += 64) {
    const int c = v2_work_units(p.seq_lens[i]);
    tot_units += c;
    before += i < b ? c : 0;
  }
  tot_units = __builtin_amdgcn_readfirstlane(wave_sum_i32(tot_units));
  before = __builtin_amdgcn_readfirstlane(wave_sum_i32(before));
  const int64_t G = p.num_chunks, T = tot_units;
  // does chunk c hold blocks of this sequence (units [before, before + mine), the first kSegCost of them start-up)?
  auto holds_blocks = [&](int64_t c) -> bool {
    const int64_t cb = c * T / G, ce = (c + 1) * T / G;
    const int64_t lo = cb > before ? cb : before, hi = ce < before + mine ? ce : before + mine;
    int64_t rlo = lo - before - kSegCost, rhi = hi - before - kSegCost;
    rlo = rlo < 0 ? 0 : rlo;
    rhi = rhi < 0 ? 0 : rhi;
    return rhi > rlo;
  };

  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  float m[kRedRows], tot[kRedRows], a[kRedRows][8];
#pragma unroll
  for (int j = 0; j < kRedRows; j++) {
    m[j] = -INFINITY;
    tot[j] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) a[j][e] = 0.f;
  }
  if (mine > 0) {
    // With at least one unit per chunk every chunk between the sequence's first and last segment holds blocks of it, and
    // the split kernel left those two partial numbers behind.  Otherwise (tiny workloads) some chunks are empty and the
    // chunk boundaries are worked out here: chunk c starts at unit floor(c*T/G), the chunk holding unit x is the
    // largest c with c*T < (x+1)*G.
    const bool dense_chunks = T >= G;
    int c, c_last;
    if (dense_chunks) {
      c = id_first - b;
      c_last = id_last - b;
    } else {
      c = (int)((((int64_t)before + 1) * G - 1) / T);
      c_last = (int)((((int64_t)before + mine) * G - 1) / T);
    }
    // wide: wavefront w takes the chunks c + w, c + w + 4, ...; where chunks have to be tested one by one (tiny
    // workloads, a handful of partials) wavefront 0 takes them all
    int c_step = 1;
    if constexpr (kWide) {
      if (dense_chunks) { c += wave; c_step = 4; }
      else if (wave != 0) c = c_last + 1;
    }
    while (c <= c_last) {
      int64_t part[kRedParts];                               // partial numbers of this pass (uniform), -1 = none
      int np = 0;
#pragma unroll
      for (int q = 0; q < kRedParts; q++) {
        while (c <= c_last && !dense_chunks && !holds_blocks(c)) c++;     // wrote nothing for this sequence
        part[q] = c <= c_last ? (int64_t)(c + b) * r_max + row0 : -1;
        if (c <= c_last) { np++; c += c_step; }
      }
      // The per-row records (log-sum-exp, correction factor, address of the dominant key's latent vector) are uniform:
      // scalar loads.  One-wavefront form: once they are here the partials AND the latent vectors of the flagged segments
      // are asked for together, so that the whole pass costs one vector-memory round trip (measured: asking for the
      // partials first costs it registers and 4 us).  Wide form: the partials are asked for first, their addresses
      // need nothing but the chunk list, and the records travel at the same time.
      h8 v[kRedRows][kRedParts];
      auto ask_partials = [&] {
#pragma unroll
        for (int q = 0; q < kRedParts; q++)
#pragma unroll
          for (int j = 0; j < kRedRows; j++) {
            const bool on = q < np && row0 + j < rows;
            const int64_t pr = on ? part[q] + j : 0;
            v[j][q] = *(const h8*)(p.o_part + pr * kDNope + lane * 8);
          }
      };
      if constexpr (kWide) ask_partials();
      float lse[kRedRows][kRedParts], cs[kRedRows][kRedParts];
      const __bf16* cp[kRedRows][kRedParts];
#pragma unroll
      for (int q = 0; q < kRedParts; q++)
#pragma unroll
        for (int j = 0; j < kRedRows; j++) {
          const bool on = q < np && row0 + j < rows;
          const int64_t pr = on ? part[q] + j : 0;
          lse[j][q] = on ? p.lse_part[pr] : -INFINITY;
          cs[j][q] = on ? p.corr_scale[pr] : 0.f;
          cp[j][q] = p.corr_row[pr];
          if (lse[j][q] == INFINITY || lse[j][q] == -INFINITY) cs[j][q] = 0.f;
        }
      if constexpr (!kWide) ask_partials();
      bf16x8 kv[kRedRows][kRedParts];
#pragma unroll
      for (int q = 0; q < kRedParts; q++)
#pragma unroll
        for (int j = 0; j < kRedRows; j++)
          if (cs[j][q] != 0.f) kv[j][q] = *(const bf16x8*)(cp[j][q] + lane * 8);
#pragma unroll
      for (int q = 0; q < kRedParts; q++)
#pragma unroll
        for (int j = 0; j < kRedRows; j++) {
          float l = lse[j][q];
          if (l == INFINITY || l == -INFINITY) continue;     // nothing visible in that segment (or no such partial)
          const float mn = fmaxf(m[j], l);
          const float so = __expf(m[j] - mn), w = __expf(l - mn);   // m = -inf at first: exp(-inf) = 0 rescales the zeros
          m[j] = mn;
          tot[j] = tot[j] * so + w;
#pragma unroll
          for (int e = 0; e < 8; e++) a[j][e] = a[j][e] * so + (float)v[j][q][e] * w;
          // the split kernel rounded this segment's dominant probability to bf16: put the difference back
          if (cs[j][q] != 0.f) {
#pragma unroll
            for (int e = 0; e < 8; e++) a[j][e] += (float)kv[j][q][e] * (w * cs[j][q]);
          }
        }
    }
  }
  if constexpr (kWide) {
    static_assert(!kWide || kRedRows == 1, "the exchange below holds one row per wavefront");
    if (lane == 0) { comb_ml[wave * 2] = m[0]; comb_ml[wave * 2 + 1] = tot[0]; }
#pragma unroll
    for (int e = 0; e < 8; e++) comb_a[(wave * 8 + e) * 64 + lane] = a[0][e];
    __syncthreads();
    if (wave == 0) {
      float mm = -INFINITY;
#pragma unroll
      for (int w = 0; w < 4; w++) mm = fmaxf(mm, comb_ml[w * 2]);
      float tt = 0.f, aa[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < 4; w++) {
        const float mw = comb_ml[w * 2];
        const float f = mw == -INFINITY ? 0.f : __expf(mw - mm);          // a wavefront without partials weighs nothing
        tt += comb_ml[w * 2 + 1] * f;
#pragma unroll
        for (int e = 0; e < 8; e++) aa[e] += comb_a[(w * 8 + e) * 64 + lane] * f;
      }
      m[0] = mm;
      tot[0] = tt;
#pragma unroll
      for (int e = 0; e < 8; e++) a[0][e] = aa[e];
    }
    __syncthreads();                                          // the exchange area is reused by the next row
    if (wave != 0) continue;
  }
#pragma unroll
  for (int j = 0; j < kRedRows; j++) {
    const int row = row0 + j;
    if (row >= rows) break;
    const int t_local = row / p.num_heads;
    const int head = row - t_local * p.num_heads;
    const float inv = tot[j] > 0.f ? 1.f / tot[j] : 0.f;
    __bf16* out = p.out + (int64_t)(q0 + t_local) * p.out_st + (int64_t)head * p.out_sh;
    bf16x8 o8;
#pragma unroll
    for (int e = 0; e < 8; e++) o8[e] = (__bf16)(a[j][e] * inv);
    *(bf16x8*)(out + lane * 8) = o8;
    if (p.lse_out && lane == 0)
      p.lse_out[(int64_t)(q0 + t_local) * p.lse_st + head] = tot[j] > 0.f ? __logf(tot[j]) + m[j] : -INFINITY;
  }
  }  // row groups of this wavefront
}

int launch_chunk_reduce(const ChunkReduceParams& p, hipStream_t stream) {
  const int64_t r_max = (int64_t)p.max_q_len * p.num_heads;
  const int64_t per_seq = p.batch > 0 ? p.num_chunks / p.batch + 1 : 0;     // about that many partials per sequence
  // many partials: past two passes of the one-wavefront form the wide form wins, as long as all rows' workgroups are
  // resident at once (two per CU at its register use)
  const bool wide = per_seq > 2 * kRedPartsNarrow && (int64_t)p.batch * r_max <= 512;
  // one or two partials and rows for more than one round of resident wavefronts: four rows per wavefront
  const bool few = !wide && per_seq <= kRedPartsFew && (int64_t)p.batch * r_max > 16384;
  if (wide) {
    const int64_t row_groups = (int64_t)p.batch * r_max;
    const int64_t wgs = row_groups < (1ll << 30) ? row_groups : (1ll << 30);
    hipLaunchKernelGGL((mla_chunk_reduce_kernel<true, false>), dim3((unsigned)wgs), dim3(256), 0, stream, p);
  } else if (few) {
    const int64_t row_groups = (int64_t)p.batch * ((r_max + kRedRowsFew - 1) / kRedRowsFew);
    hipLaunchKernelGGL((mla_chunk_reduce_kernel<false, true>), dim3((unsigned)((row_groups + 3) / 4)), dim3(256), 0, stream, p);
  } else {
    const int64_t row_groups = (int64_t)p.batch * r_max;
    hipLaunchKernelGGL((mla_chunk_reduce_kernel<false, false>), dim3((unsigned)((row_groups + 3) / 4)), dim3(256), 0, stream, p);
  }
  return check_launch("mla_chunk_reduce_kernel");
}

int launch_decode_v2(const DecodeV2Params& p, bool sparse, dim3 grid, hipStream_t stream) {
  const int rc = sparse ? ensure_dynamic_lds((const void*)mla_decode_v2_kernel<true, false>, kV2LdsB, "dsa_sparse_decode_bf16")
                        : ensure_dynamic_lds((const void*)mla_decode_v2_kernel<false, false>, kV2LdsB, "mla_decode_bf16");
  if (rc != MLA_OK) return rc;
  if (sparse) hipLaunchKernelGGL((mla_decode_v2_kernel<true, false>), grid, dim3(256), kV2LdsB, stream, p);
  else hipLaunchKernelGGL((mla_decode_v2_kernel<false, false>), grid, dim3(256), kV2LdsB, stream, p);
  return check_launch("mla_decode_v2_kernel");
}

int launch_decode_v2_window(const DecodeV2Params& p, dim3 grid, hipStream_t stream) {
  const int rc = ensure_dynamic_lds((const void*)mla_decode_v2_kernel<false, true>, kV2LdsB, "mla_decode_bf16_window_split");
  if (rc != MLA_OK) return rc;
  hipLaunchKernelGGL((mla_decode_v2_kernel<false, true>), grid, dim3(256), kV2LdsB, stream, p);
  return check_launch("mla_decode_v2_kernel");
}

}  // namespace mlahip
