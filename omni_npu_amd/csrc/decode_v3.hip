// Absorbed-MLA paged decode over the bf16 cache: split-KV kernel with eight wavefronts per workgroup (two per SIMD).
//
// Contract: the reference's decode call (src/omni_npu/attention/backends/mla.py:781-804); dense paged source, per-token
// row lists (src/omni_npu/attention/backends/dsa.py:259-291) and the sink + sliding-window variant
// (src/omni_npu/attention/backends/mla.py:705-779) are instantiations of one kernel.
//
// A query row is a (token, head) pair; a workgroup handles 128 rows and streams 32-key blocks of the latent cache
// through LDS.  With one 512-register wavefront per SIMD every instruction of the block loop is issued in series and the
// matrix pipe idles during each LDS read, softmax instruction and wait; with two 256-register wavefronts per SIMD the
// other wavefront's MFMAs fill those gaps, and the CU's LDS read rate doubles (a wavefront cannot draw more than ~32 B
// per clock by itself).  The register file holds the same data either way: 256 KiB of fp32 output accumulators and
// 144 KiB of query, spread over eight wavefronts:
//   S^T = K Q^T      wave w owns query rows 16w..16w+15 (its 576-wide query stays in 72 registers) and all 32 keys of a
//                    block: 36 v_mfma_f32_16x16x32_bf16, one 16-byte LDS row read (the K fragment) each;
//   O^T += V^T P^T   wave w owns output columns [64w, 64w+64) for ALL 128 rows (128 accumulation registers): 16
//                    v_mfma_f32_32x32x16_bf16 per block, V^T fragments by transposed LDS reads of the same rows.
// P^T (bf16) travels through LDS once per block (8 KiB, double buffered), one workgroup barrier per block.
//
// Pipeline:  body i = [barrier] the copies of block i+3 (wavefronts 0..3), QK(i+1) | PV(i) with the softmax of
// block i+1 cut into steps between the MFMA groups | publish P(i+1).
//
// Softmax with a fixed reference (no accumulator rescaling: vector ALU instructions cannot touch the accumulation
// registers): every row fixes m_ref at the largest score of its first block and uses P = exp2(s - m_ref) from then on;
// bf16 and fp32 share an exponent range, so P may grow to 2^100 without loss of relative precision.  A score more than
// 100 (log2) above the reference raises a flag; the workgroup then restarts its segment with the maxima seen so far.
// In the steady state nothing crosses lanes: the four lanes that hold a row's scores keep their own sums and candidates
// for the row's most probable key, and combine them in the epilogue.
// Partials: normalised fp16 through an LDS transpose, fp32 natural-log LSE, and the dominant-key correction record that
// mla_chunk_reduce_kernel applies (the bf16 rounding of the largest probability is the biggest single error of P.V).
#include "decode_params.hpp"
#include <type_traits>
#include <cstdlib>

namespace mlahip {
namespace v3 {

constexpr int kBlk = 32;                                   // keys per block
constexpr int kNopeBufB = kBlk * 1024;                     // 32768
constexpr int kRopeBufB = kBlk * 128;                      // 4096
constexpr int kRopeOff = 4 * kNopeBufB;                    // 131072
constexpr int kPOff = kRopeOff + 3 * kRopeBufB;            // 143360
constexpr int kPBufB = 8192;                               // 4 row groups x 2 k-blocks x 64 lanes x 16 B
constexpr int kFlagOff = kPOff + 2 * kPBufB;               // 159744: restart flags, 2 x 8 dwords
constexpr int kLimitOff = kFlagOff + 64;                   // per row of the group: number of visible keys (read by masking blocks only)
constexpr int kSeenOff = kLimitOff + 512;                  // per lane: the score that raised its restart flag
constexpr int kKTabOff = kSeenOff + 2048;                  // per lane: LDS offsets of its K-fragment reads (latent, rope)
constexpr int kIdsOff = kKTabOff + 512;                    // row lists: 4 blocks x 4 copying waves x the wave's eight cache rows
constexpr int kLdsB = kIdsOff + 512;
static_assert(kLdsB <= 160 * 1024, "LDS budget");
constexpr int kLead = 3;                                   // block i + kLead is copied while block i is consumed
constexpr int kCopyWaves = 4;                              // wavefronts 0..3 issue the copies (the older wavefront of each SIMD)
constexpr int kCopies = 9;                                 // copy instructions per copying wavefront and block (8 nope rows + rope)
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


// kRG = groups of 32 query rows a workgroup handles (4: the general form; 1 or 2: launches with at most 32 / 64 query rows
// per request, e.g. the 16 heads a tensor-parallel rank of eight owns, and row-list launches whose chunks alone would
// leave most of the CUs idle, which then give every 32 or 64 rows a workgroup of their own: blockIdx.z).  With few rows the 128-row schedule spends the same
// MFMAs, LDS reads and watts on rows that do not exist, so the small forms leave them out: only the wavefronts that own
// rows run the S phase and the softmax, P.V covers kRG row groups, and the copies move to wavefronts 4..7, which have
// nothing else to do in the S phase.  The kernel is then bound by the cache stream alone.
template <bool kSparse, bool kWindow, int kRG = 4, bool kWrite = false>
__global__ __launch_bounds__(512) void mla_decode_v3_kernel(const DecodeParams p) {
  static_assert(!(kSparse && kWindow), "the window variant reads the paged cache");
  static_assert(!kWrite || (!kSparse && !kWindow), "the folded cache write belongs to the dense kernel");
  static_assert(kRG == 1 || kRG == 2 || kRG == 4, "row groups");
  constexpr int kGrpRows = 32 * kRG;                          // query rows of one workgroup (blockIdx.z counts such groups)
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
  if constexpr (kWrite) {
    // The step's cache write, folded in: the rows of this request's query tokens are the keys L - qlen .. L - 1; those
    // that lie in this segment's blocks are stored now (token j by wavefront j: 64 lanes x 16 bytes of latent, 8 lanes of
    // rope), and every store has been acknowledged before any wavefront asks for a block.  Each key belongs to exactly
    // one chunk, so a row is written by the workgroups that are going to read it and by nobody else (with more than 128
    // query rows the row groups of the chunk each store the same bytes: none of them may read before its own store).
    {
      KernArgPtr kp = cold();
      for (int j = wave; j < qlen; j += 8) {
        const int pos = L - qlen + j;
        if (pos < blk_begin * kBlk || pos >= blk_end * kBlk) continue;
        const int64_t slot = kp->new_slots[q0 + j];
        if (slot < 0 || slot >= kp->num_pages * kPage) continue;
        const int64_t pg = slot / kPage, off = slot - pg * kPage;
        const u32x4 vn = *(const u32x4*)(kp->new_c + (int64_t)(q0 + j) * kp->new_c_st + lane * 8);
        *(u32x4*)(const_cast<__bf16*>(kp->nope) + pg * kp->nope_sp + off * kp->nope_sr + lane * 8) = vn;
        if (lane < 8) {
          const u32x4 vr = *(const u32x4*)(kp->new_r + (int64_t)(q0 + j) * kp->new_r_st + lane * 8);
          *(u32x4*)(const_cast<__bf16*>(kp->rope) + pg * kp->rope_sp + off * kp->rope_sr + lane * 8) = vr;
        }
      }
      MLA_WAIT_VMCNT(0);
    }
    lds_barrier();
  }
  const int rows = qlen * p.num_heads;
  const bool has_rows = kRG == 4 || (wave * 16 < kGrpRows && grp * kGrpRows + wave * 16 < rows);

  // this lane's query row for QK / softmax; the four lanes l16 + 16*g share it
  const int rloc = wave * 16 + l16;                           // row inside the group (the small forms use the first kGrpRows)
  const int row = grp * kGrpRows + rloc;
  const bool row_ok = row < rows && rloc < kGrpRows && L > 0;
  const int t_local = row / p.num_heads;
  const int head = row - t_local * p.num_heads;
  {
    int limit = row_ok ? (L - qlen + t_local + 1) : 0;       // keys [0, limit) are visible to this row
    limit = limit < 0 ? 0 : limit;
    if (g == 0) *(int*)(lds + kLimitOff + rloc * 4) = limit;  // read back by the blocks that have to mask (the last ones)
    *(float*)(lds + kSeenOff + threadIdx.x * 4) = -INFINITY;
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

  // ---- global -> LDS copies: wavefronts 0..3 copy eight nope rows (1 KiB each) and eight rope rows per block ----
  // A copy instruction stalls at issue while the memory pipeline is full, and a stalled wavefront issues nothing else.
  // The two wavefronts of a SIMD (w and w + 4) would stall at the same moments if both copied; with all copies in the
  // older one the younger one keeps the matrix pipe busy meanwhile, and the older one is the one that otherwise waits
  // at the barrier.
  // Row r of a block goes to nope buffer row r (granule gr at position gr ^ swz(r)) and rope buffer row r.  Wave w copies
  // rows 8w..8w+7: swz(8w + j) = swz(8w) ^ swz(j), so one per-lane offset serves all eight rows.
  // The per-lane offsets are worked out from the hardware lane number at every use (a handful of vector ALU
  // instructions per block, in the phase where that unit idles) instead of occupying registers through the loop.
  const uint32_t n_sr2 = (uint32_t)p.nope_sr * 2u, r_sr2 = (uint32_t)p.rope_sr * 2u;       // row strides in bytes
  const bool copier = kRG == 4 ? wave < kCopyWaves : wave >= 8 - kCopyWaves;
  const int cw = kRG == 4 ? wave : (wave & 3);                // the copying wavefront's number among the four
  const int swz_nw = swz_nope((cw * 8) & 15), swz_rw = swz_rope((cw * 8) & 15);            // scalars
  // full blocks of the paged cache: the wave's row offsets ride in the per-lane offset (32 rows stay below 2^31 bytes,
  // checked where the mode is chosen), so a copy is one vector instruction, one scalar add into M0 and the load
  const bool full_ok = n_sr2 <= (1u << 25) && r_sr2 <= (1u << 25);
  const uint32_t dma_off = (uint32_t)((lane ^ swz_nw) << 4);
  uint32_t s_rowoff[8];
#pragma unroll
  for (int k = 0; k < 8; k++) s_rowoff[k] = (uint32_t)(cw * 8 + k) * n_sr2;

  ConstI32Ptr bt = (ConstI32Ptr)(p.block_table) + (kSparse ? 0 : (int64_t)b * p.bt_stride);
  const int64_t max_row = p.num_pages * p.page_size - 1;
  // The hardware lane number behind an opaque (and volatile) statement: what is derived from it inside the loop is
  // computed inside the loop.  Left alone the compiler hoists every loop-invariant LDS address out of the block loop, a
  // dozen registers of them, and then spills them - and a scratch reload waits for every copy in flight.
  auto lane_now = [] {
    int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(ln));
    return ln;
  };
  // Row list (kSparse): a wave copies rows 8w..8w+7 of a block and needs the cache rows of exactly those eight keys.  They
  // are fetched one block ahead by an eight-lane global -> LDS copy into the wave's own slot (no register is the target of
  // a load in flight, so nothing the compiler does with registers in between can lose them), issued in front of the
  // copies of the previous block so that the wait that lets those land covers it, and read back when the copies are due.
  // Keys past the end of the list name its last key (their scores are masked).
  int32_t ids_rope = 0;                                       // cache row of this lane's rope row
  int32_t ids_row[8] = {0, 0, 0, 0, 0, 0, 0, 0};              // cache rows of the wave's eight keys (uniform)
  auto ids_dma = [&](int blk_x) {
    if constexpr (kSparse) {
      if (copier) {
        int tok = blk_x * kBlk + cw * 8 + (lane_now() & 7);
        tok = tok < L ? tok : L - 1;
        tok = tok < 0 ? 0 : tok;
        dma4_sv_lanes8(p.sparse_rows + (int64_t)b * p.sparse_stride, (uint32_t)tok * 4u, lds0 + kIdsOff + (blk_x & 3) * 128 + cw * 32);
      }
    }
  };
  auto ids_fetch = [&](int blk_x) {
    if constexpr (kSparse) {
      if (copier) {
        const int ln = lane_now();
        const char* slot = lds + kIdsOff + (blk_x & 3) * 128 + cw * 32;
        const int32_t mine = *(const int32_t*)(slot + (ln & 7) * 4);
        ids_rope = *(const int32_t*)(slot + ((ln >> 3) & 7) * 4);
#pragma unroll
        for (int k = 0; k < 8; k++) ids_row[k] = __builtin_amdgcn_readlane(mine, k);
      }
    }
  };
  auto load_page = [&](int page) -> int64_t {
    page = page < p.max_blocks ? page : p.max_blocks - 1;
    int64_t pg = bt[page];
    return pg < 0 ? 0 : (pg >= p.num_pages ? p.num_pages - 1 : pg);
  };
  int page_cur = 0;
  int64_t pg_nxt = 0;
  // Blocks are copied in order, so the address of the next block's first row is a running pointer: 32 rows further
  // inside a page, recomputed (64-bit products) only where a new page starts.
  const char* np_blk = (const char*)p.nope;
  const char* rp_blk = (const char*)p.rope;
  const uint64_t n_blk_b = (uint64_t)n_sr2 * kBlk, r_blk_b = (uint64_t)r_sr2 * kBlk;
  auto set_page = [&](int64_t pg, int cblk) {
    np_blk = (const char*)p.nope + pg * p.nope_sp * 2 + (uint64_t)((cblk & 3) * kBlk) * n_sr2;
    rp_blk = (const char*)p.rope + pg * p.rope_sp * 2 + (uint64_t)((cblk & 3) * kBlk) * r_sr2;
  };
  auto issue_reset = [&]() {
    if constexpr (!kSparse) {
      const int cblk = blk_begin + (kWindow && blk_begin >= win_blk0 ? win_skip : 0);
      page_cur = cblk >> 2;
      set_page(load_page(page_cur), cblk);
      pg_nxt = load_page(page_cur + 1);
    }
  };
  // The nine copies of a block ("pieces").  Rows past the end of the sequence re-read its last row (their scores are masked).
  // rope buffer of a block: (blk - blk_begin + rope_ph) % 3 without a division (rope_ph = blk_begin % 3 once per segment)
  const int rope_ph = blk_begin % 3;
  auto rope_buf_of = [&](int blk) -> int {
    int r = (blk - blk_begin + rope_ph);                      // counts up by one per block from a value below 3
    r -= 3 * (int)(((uint32_t)r * 43691u) >> 17);             // r / 3 for r < 98304: one multiply, no division sequence
    return r;
  };
  struct IssueCtx { const char* np; const char* rp; uint32_t nbuf, rbuf; int last, tok0; };
  auto issue_begin = [&](int blk) -> IssueCtx {
    IssueCtx c;
    c.tok0 = blk * kBlk;
    c.last = L - 1 - c.tok0;                                  // last valid row of the block (>= 0)
    c.nbuf = lds0 + (blk & 3) * kNopeBufB;
    c.rbuf = lds0 + kRopeOff + rope_buf_of(blk) * kRopeBufB;
    if constexpr (kSparse) {
      c.np = (const char*)p.nope;
      c.rp = (const char*)p.rope;
    } else {
      const int cblk = blk + (kWindow && blk >= win_blk0 ? win_skip : 0);   // block of the cache
      const int page = cblk >> 2;
      if (page != page_cur) {
        // the next page's number is only asked for here (raw: clamping it now would wait for the load); it is clamped
        // when it becomes the current page, four blocks later
        if (kWindow && page != page_cur + 1) set_page(load_page(page), cblk);  // the jump from the sink to the window
        else set_page(pg_nxt < 0 ? 0 : (pg_nxt >= p.num_pages ? p.num_pages - 1 : pg_nxt), cblk);
        page_cur = page;
        const int pn = page + 1 < p.max_blocks ? page + 1 : p.max_blocks - 1;
        pg_nxt = bt[pn];
      }
      c.np = np_blk;
      c.rp = rp_blk;
      np_blk += n_blk_b;
      rp_blk += r_blk_b;
    }
    return c;
  };
  auto rope_lane_row = [&] { return (lane_now() >> 3) & 7; };                               // lane's row among the wave's eight
  auto rope_lane_off = [&]() -> uint32_t {
    const int ln = lane_now(), t = (ln >> 3) & 7;
    return (uint32_t)(((ln & 7) ^ swz_rw ^ ((t & 1) << 2) ^ (t & 2) ^ (t >> 2)) << 4);      // swz_rope(t) = (t0 << 2) | (t1 << 1) | t2
  };
  // kFull: every row of the block exists and the source is the paged cache
  // When a chunk's cache rows are read by this workgroup alone (one group of query rows per chunk) they are read once in
  // the whole launch, and the copies are marked non-temporal: 1-2 us of 120 on the headline shape.  With several row
  // groups per chunk the groups find each other's rows in the XCD's L2, and the mark costs that (16 short sequences in
  // groups of 32 rows: 30.1 -> 33.7 us), so it is left off there.
  const bool stream_once = !kSparse && gridDim.z == 1;
  // kNt: the copy is marked non-temporal
  auto issue_piece = [&](IssueCtx& c, int k, auto full, auto nt) {
    constexpr bool kFull = decltype(full)::value && !kSparse;
    constexpr bool kNt = decltype(nt)::value && !kSparse;
    auto clampi = [&](int64_t s_) -> int64_t { return s_ < 0 ? 0 : (s_ > max_row ? max_row : s_); };

    if (k < 8) {
      const int r = cw * 8 + k;
      if constexpr (kFull) {
        uint32_t d = dma_off;
        asm volatile("" : "+v"(d));                           // (opaque: the eight offsets are not precomputed and spilled)
        if constexpr (kNt) dma16_sv_m0add_nt(c.np, (d ^ (uint32_t)(swz_nope(k) << 4)) + s_rowoff[k], c.nbuf + cw * 8192, k * 1024);
        else dma16_sv_m0add(c.np, (d ^ (uint32_t)(swz_nope(k) << 4)) + s_rowoff[k], c.nbuf + cw * 8192, k * 1024);
      } else {
        const uint32_t off = (uint32_t)((lane_now() ^ swz_nw ^ swz_nope(k)) << 4);
        const int re = r < c.last ? r : c.last;
        if constexpr (kSparse) dma16_sv(c.np + clampi(ids_row[k]) * n_sr2, off, c.nbuf + r * 1024);
        else if constexpr (kNt) dma16_sv_nt(c.np + (uint64_t)re * n_sr2, off, c.nbuf + r * 1024);
        else dma16_sv(c.np + (uint64_t)re * n_sr2, off, c.nbuf + r * 1024);
      }
    } else {
      // the wave's eight rope rows, 128 bytes each: one instruction
      if constexpr (kSparse) {
        dma16_v(c.rp + clampi(ids_rope) * r_sr2 + rope_lane_off(), c.rbuf + cw * 1024);
      } else if constexpr (kFull) {
        if constexpr (kNt) dma16_sv_nt(c.rp, (uint32_t)(cw * 8 + rope_lane_row()) * r_sr2 + rope_lane_off(), c.rbuf + cw * 1024);
        else dma16_sv(c.rp, (uint32_t)(cw * 8 + rope_lane_row()) * r_sr2 + rope_lane_off(), c.rbuf + cw * 1024);
      } else {
        const int r = cw * 8 + rope_lane_row();
        const int re = r < c.last ? r : c.last;
        if constexpr (kNt) dma16_sv_nt(c.rp, (uint32_t)re * r_sr2 + rope_lane_off(), c.rbuf + cw * 1024);
        else dma16_sv(c.rp, (uint32_t)re * r_sr2 + rope_lane_off(), c.rbuf + cw * 1024);
      }
    }
  };
  auto issue_block = [&](int blk) {
    IssueCtx c = issue_begin(blk);
    if (copier) {
#pragma unroll
      for (int k = 0; k < kCopies; k++) issue_piece(c, k, std::false_type{}, std::false_type{});
    }
  };
  // Row list: the rows of the first kLead blocks are fetched together (one round trip) before any copy goes out
  auto issue_first = [&]() {
    issue_reset();
    if constexpr (kSparse) {
#pragma unroll
      for (int j = 0; j < kLead; j++) ids_dma(blk_begin + j);
      MLA_WAIT_VMCNT(0);
      ids_fetch(blk_begin);
    }
    issue_block(blk_begin);
  };
  auto issue_next_two = [&]() {
#pragma unroll 1
    for (int j = 1; j < kLead && j < nb; j++) {
      ids_fetch(blk_begin + j);
      issue_block(blk_begin + j);
    }
  };

  // ---- prologue: the query, then the first blocks' copies ----
  // The MFMA operand layout wants, per load instruction, 16 bytes of 64 different cache lines: read straight from
  // memory the texture addresser needs 64 cycles per instruction and the query takes ten microseconds.  So every wave
  // copies its own 16 rows global -> LDS whole (one row per instruction, into the tile buffers, which are free at the
  // start of a segment) and picks its operands from there.  The copies of the first key blocks have to wait until
  // every wave has its query in registers (one barrier).
  bf16x8 qf[18];                                             // contraction steps of 32: 16 over the latent part, 2 over rope
  // One row group: the two wavefronts that can own rows stage their query in the tile buffer of the segment's FOURTH block,
  // which is not requested before the block loop runs, so the copying wavefronts ask for the first three blocks now and
  // the query's round trip to memory hides under theirs.
  const uint32_t q_stage = kRG == 1 ? (uint32_t)(((blk_begin + 3) & 3) * kNopeBufB) : 0u;
  if (!has_rows) {
#pragma unroll
    for (int kk = 0; kk < 18; kk++) qf[kk] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (kRG == 1) {
      issue_first();
      ids_dma(blk_begin + kLead);
      issue_next_two();
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
        dma16_sv(src, (uint32_t)((ln ^ swz_nope(k)) << 4), lds0 + q_stage + wave * 16384 + k * 1024);
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
    for (int kk = 0; kk < 16; kk++) qf[kk] = *(const bf16x8*)(lds + q_stage + (qoff ^ (uint32_t)((kk >> 2) << 4)) + (kk & 3) * 256);
#pragma unroll
    for (int kk = 0; kk < 2; kk++) qf[16 + kk] = *(const bf16x8*)(lds + kPOff + wave * 2048 + ql16 * 128 + (2 * qg + kk) * 16);
#pragma unroll
    for (int kk = 0; kk < 18; kk++) asm volatile("" : "+v"(qf[kk]));           // the query stays in VGPRs
  }
  lds_barrier();                                              // every wave has read its query: the tile buffers are free
  if constexpr (kRG != 1) issue_first();

  f32x16 acc[2][4];                                          // [32-column block of this wave's 64][row group]
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  float m_ref = -INFINITY;       // the row's softmax reference (log2 domain), the same in its four lanes
  float l_run = 0.f;             // this lane's share of the row's sum
  float top_p = 0.f;             // largest probability among this lane's visible keys so far ...
  int top_tag = -1;              // ... and where: (block << 3) | element number

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
  auto qk_block = [&](int blk, f32x4 (&s)[2], auto issue, int blk_issue) {
    constexpr int kIssueMode = decltype(issue)::value;       // 0: no copies; 1: any block; 2: a full block of the paged cache
    constexpr bool kIssue = kIssueMode != 0;
    // the six addresses the 36 reads use (the rest is immediate offsets)
    uint32_t na[4], ra[2];
    const u32x2 kr = *(const u32x2*)(lds + kKTabOff + lane_now() * 8);
    na[0] = lds0 + (blk & 3) * kNopeBufB + kr[0];
    ra[0] = lds0 + rope_buf_of(blk) * kRopeBufB + kr[1];
#pragma unroll
    for (int b4 = 1; b4 < 4; b4++) na[b4] = na[0] ^ (uint32_t)(b4 << 4);
    ra[1] = ra[0] ^ 16u;
    IssueCtx ic;
    if constexpr (kIssue) { ids_dma(blk_issue + 1); ic = issue_begin(blk_issue); }
    // All nine copies go out here, in front of the wave's K reads: the copying wave then runs its S phase a few hundred
    // clocks behind the other wave of its SIMD (which copies nothing), and the two want the LDS and the matrix pipe at
    // different moments (measured against the copies spread between the MFMAs: 121.8 / 123.4 -> 119.5 / 121.5 us).
    if constexpr (kIssue) {
      if (stream_once) {
#pragma unroll
        for (int k = 0; k < kCopies; k++) issue_piece(ic, k, std::integral_constant<bool, kIssueMode == 2>{}, std::true_type{});
      } else {
#pragma unroll
        for (int k = 0; k < kCopies; k++) issue_piece(ic, k, std::integral_constant<bool, kIssueMode == 2>{}, std::false_type{});
      }
    }
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
  // vector work behind the MFMAs), and it is kept to the minimum: per score one tag, one FMA, one exponential, one add,
  // half a conversion.  The lane's eight raw scores (key 16*(r/4) + 4g + r%4 at sc[r]) first get their element number r
  // into the three low mantissa bits (7 ulp: 1e-5 of a probability), so the float maximum of the tagged scores names
  // the lane's most probable key and its probability without a second pass over the probabilities.
  // Nothing here crosses lanes: sums and dominant-key candidates are per lane and are combined in the epilogue.
  struct Sm { float t, pm, psum; uint32_t mx; uint32_t pw[4]; };   // t = scaled max score - reference (log2), pm = exp2(t); pw: bf16 pairs
#define SM_TAG(r) asm volatile("v_and_or_b32 %0, %0, -8, %1" : "+v"(sc[r]) : "n"(r))
#define SM_EXP2(a, b)                                                                                                   \
  asm volatile("v_fma_f32 %0, %0, %2, -%3\n\tv_fma_f32 %1, %1, %2, -%3\n\tv_exp_f32 %0, %0\n\tv_exp_f32 %1, %1"          \
               : "+v"(sc[a]), "+v"(sc[b]) : "s"(p.scale_log2), "v"(m_ref))
  auto sm_head = [&](float (&sc)[8], Sm& st) {               // tags and the lane's maximum (12 instructions)
    SM_TAG(0); SM_TAG(1); SM_TAG(2); SM_TAG(3); SM_TAG(4); SM_TAG(5); SM_TAG(6); SM_TAG(7);
    asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(st.mx) : "v"(sc[0]), "v"(sc[1]), "v"(sc[2]));
    asm volatile("v_max3_f32 %0, %0, %1, %2\n\tv_max3_f32 %0, %0, %3, %4\n\tv_max_f32 %0, %0, %5"
                 : "+v"(st.mx) : "v"(sc[3]), "v"(sc[4]), "v"(sc[5]), "v"(sc[6]), "v"(sc[7]));
  };
  auto sm_pm = [&](Sm& st) {
    asm volatile("v_fma_f32 %0, %2, %3, -%4\n\ts_nop 0\n\tv_exp_f32 %1, %0\n\ts_nop 0" : "=&v"(st.t), "=v"(st.pm) : "v"(st.mx), "s"(p.scale_log2), "v"(m_ref));
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
    const uint32_t vb = lds0 + (blk & 3) * kNopeBufB;
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
    // The small forms have matrix time to spare and spend it on precision: a probability goes through P.V as TWO bf16
    // numbers, its rounded value and the rounding's remainder (fragments rg + 2 of the exchange buffer), each fragment of
    // V^T feeding both.  The product then carries 16 significant bits of every probability instead of 8, and the result's
    // error is the rounding of the output alone.
    if constexpr (kRG == 1) {
      // one row group: four MFMAs per k-block, the softmax steps in the shadow of the LDS reads
      if constexpr (kPv) { PV_VREAD(0); PV_PREAD(pr0, 0, 0); PV_PREAD(pr1, 2, 0); }
      if constexpr (kSm) { if (sm_on) { sm_head(sc, st); SM_EXP2(0, 1); SM_EXP2(2, 3); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_MFMA2(0, pr1, 0); PV_VREAD(1); PV_PREAD(pr0, 0, 1); PV_PREAD(pr1, 2, 1); }
      if constexpr (kSm) { if (sm_on) { SM_EXP2(4, 5); SM_EXP2(6, 7); sm_pm(st); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_MFMA2(0, pr1, 0); PV_SETTLE(0); }
      if constexpr (kSm) { if (sm_on) { sm_sum_lo(sc, st); sm_sum_hi(sc, st); } }
    } else if constexpr (kRG == 2) {
      // (two register quads for the four P^T fragments of a k-block, each refilled as soon as its MFMAs are issued)
      if constexpr (kPv) { PV_VREAD(0); PV_PREAD(pr0, 0, 0); PV_PREAD(pr1, 2, 0); }
      if constexpr (kSm) { if (sm_on) { sm_head(sc, st); SM_EXP2(0, 1); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_PREAD(pr0, 1, 0); PV_MFMA2(0, pr1, 1); PV_PREAD(pr1, 3, 0); }
      if constexpr (kSm) { if (sm_on) SM_EXP2(2, 3); }
      if constexpr (kPv) { PV_MFMA2(1, pr0, 1); PV_MFMA2(1, pr1, 0); PV_VREAD(1); PV_PREAD(pr0, 0, 1); PV_PREAD(pr1, 2, 1); }
      if constexpr (kSm) { if (sm_on) { SM_EXP2(4, 5); SM_EXP2(6, 7); sm_pm(st); } }
      if constexpr (kPv) { PV_MFMA2(0, pr0, 1); PV_PREAD(pr0, 1, 1); PV_MFMA2(0, pr1, 1); PV_PREAD(pr1, 3, 1); }
      if constexpr (kSm) { if (sm_on) sm_sum_lo(sc, st); }
      if constexpr (kPv) { PV_MFMA2(1, pr0, 1); PV_MFMA2(1, pr1, 0); PV_SETTLE(0); PV_SETTLE(1); }
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
      float pv = 0.f;
      int best = 0;
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const int kpos = 16 * (r >> 2) + (r & 3);
        const float v = (kpos < rel && kpos >= rel_lo) ? sc[r] : 0.f;
        sc[r] = v;
        st.psum += v;
        best = v > pv ? r : best;
        pv = fmaxf(pv, v);
      }
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const bf16x2 pr2 = {(__bf16)sc[2 * j], (__bf16)sc[2 * j + 1]};
        st.pw[j] = __builtin_bit_cast(uint32_t, pr2);
      }
      st.pm = pv;                                             // largest VISIBLE probability of the lane in this block
      st.mx = (uint32_t)best;
    }
    // Remember the most probable key: the bf16 rounding of its probability is the largest single error of the P.V
    // product when the softmax is peaked, and the merge kernel takes it out again.
    {
      const bool nw = st.pm > top_p;
      top_p = nw ? st.pm : top_p;
      top_tag = nw ? (int)((uint32_t)(blk << 3) | (st.mx & 7u)) : top_tag;   // decoded in the epilogue
    }
    l_run += st.psum;
    const uint32_t pw = lds0 + (blk & 1) * kPBufB + p_w_off_now();
    const u32x2 w0 = {st.pw[0], st.pw[1]}, w1 = {st.pw[2], st.pw[3]};
    asm volatile("ds_write_b64 %0, %1\n\tds_write_b64 %0, %2 offset:1024" :: "v"(pw), "v"(w0), "v"(w1) : "memory");
    if constexpr (kRG < 4) {
      // what the rounding to bf16 left of every probability, as a second bf16 (row groups 2 and 3 of the buffer)
      uint32_t lo[4];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float r0 = sc[2 * j] - __builtin_bit_cast(float, st.pw[j] << 16);
        const float r1 = sc[2 * j + 1] - __builtin_bit_cast(float, st.pw[j] & 0xffff0000u);
        const bf16x2 pr2 = {(__bf16)r0, (__bf16)r1};
        lo[j] = __builtin_bit_cast(uint32_t, pr2);
      }
      const u32x2 l0 = {lo[0], lo[1]}, l1 = {lo[2], lo[3]};
      asm volatile("ds_write_b64 %0, %1 offset:4096\n\tds_write_b64 %0, %2 offset:5120" :: "v"(pw), "v"(l0), "v"(l1) : "memory");
    }
    const bool flag = st.t > kRestartThreshold;               // asks the workgroup to restart with better references
    const bool any = __builtin_amdgcn_ballot_w64(flag) != 0;
    if (any) {
      // (rare) the scores that outgrew the reference are remembered: they become the references of the restart
      float* seen = (float*)(lds + kSeenOff + (wave * 64 + lane_now()) * 4);
      if (flag) *seen = fmaxf(*seen, st.t + m_ref);
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
    // (row groups are read whole by the P.V phase; nobody else writes these slots)
    if (!has_rows) {
      const u32x2 z = {0u, 0u};
      const uint32_t pw = lds0 + p_w_off_now();
      asm volatile("ds_write_b64 %0, %1\n\tds_write_b64 %0, %1 offset:1024\n\tds_write_b64 %0, %1 offset:8192\n\tds_write_b64 %0, %1 offset:9216"
                   :: "v"(pw), "v"(z) : "memory");
      // and the slots of the remainders, two row groups further on, when this wavefront's row group is one that P.V reads
      // (the wavefronts of row groups 2 and 3 have just cleared the remainder slots of groups 0 and 1 by the lines above;
      // a barrier stands between these writes and the first published block)
      if (wave < 4)
        asm volatile("ds_write_b64 %0, %1 offset:4096\n\tds_write_b64 %0, %1 offset:5120\n\tds_write_b64 %0, %1 offset:12288\n\t"
                     "ds_write_b64 %0, %1 offset:13312" :: "v"(pw), "v"(z) : "memory");
    }
  }
  bool restart = false;
  bool early_issued = kRG == 1;  // (one row group: the first three blocks were requested beside the query)
  int restarts_left = 4;         // every restart raises a reference by more than 2^100: fp32 has room for three
  do {
    if (restart) {
      // a row outgrew its reference: drain, take the maxima seen so far as references, clear the sums, start over
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      float ms = *(const float*)(lds + kSeenOff + (wave * 64 + lane_now()) * 4);
      ms = fmaxf(ms, __shfl_xor(ms, 16, 64));
      ms = fmaxf(ms, __shfl_xor(ms, 32, 64));
      m_ref = fmaxf(m_ref, ms);
      l_run = 0.f;
      top_p = 0.f;
      top_tag = -1;
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
      issue_first();
      restart = false;
      early_issued = false;
    }
    if (!early_issued) {
      ids_dma(blk_begin + kLead);                             // (older than the copies below: their wait covers it)
      issue_next_two();
    }
    early_issued = false;
    // ---- block 0: QK, softmax, publish ----
    {
      if (nb > 2) MLA_WAIT_VMCNT(18); else if (nb > 1) MLA_WAIT_VMCNT(9); else MLA_WAIT_VMCNT(0);   // (kCopies per block in flight)
      lds_barrier();
      f32x4 s[2];
      Sm st;
      if (has_rows) {
      qk_block(blk_begin, s, std::integral_constant<int, 0>{}, 0);
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
    asm volatile("" :: "v"(vbase[0]), "v"(vbase[1]), "v"(m_ref), "v"(l_run), "v"(top_p), "v"(top_tag), "v"(dma_off));
    // ---- steady state: QK(i+1), then P.V(i) with the softmax of block i+1 riding along ----
    for (int i = 0; i + 1 < nb; i++) {
      const int blk = blk_begin + i;
      // block i+1 has landed, P(i) is published, everyone is done with P.V(i-1)
      if (i + 2 < nb) MLA_WAIT_VMCNT(9); else MLA_WAIT_VMCNT(0);
      lds_barrier();
      if (i + kLead < nb) ids_fetch(blk + kLead);             // (row list) the rows of the block whose copies go out now
      const int fl = flags_read(blk);
      f32x4 s[2];
      if constexpr (kRG < 4) {
        // small forms: wavefronts 4..7 only copy, the wavefronts that own rows only compute
        if (copier) {
          if (i + kLead < nb) {
            ids_dma(blk + kLead + 1);
            IssueCtx ic = issue_begin(blk + kLead);
            if (kSparse || !full_ok || L - 1 - (blk + kLead) * kBlk < kBlk - 1) {
#pragma unroll
              for (int k = 0; k < kCopies; k++) issue_piece(ic, k, std::false_type{}, std::false_type{});
            } else if (stream_once) {
#pragma unroll
              for (int k = 0; k < kCopies; k++) issue_piece(ic, k, std::true_type{}, std::true_type{});
            } else {
#pragma unroll
              for (int k = 0; k < kCopies; k++) issue_piece(ic, k, std::true_type{}, std::false_type{});
            }
          }
        } else if (has_rows) {
          qk_block(blk + 1, s, std::integral_constant<int, 0>{}, 0);
        }
      } else
      // (the wavefronts that copy nothing take the variant without copies: no branch around each copy, no page arithmetic)
      if (i + kLead >= nb || !copier) qk_block(blk + 1, s, std::integral_constant<int, 0>{}, 0);
      else if (kSparse || !full_ok || L - 1 - (blk + kLead) * kBlk < kBlk - 1) qk_block(blk + 1, s, std::integral_constant<int, 1>{}, blk + kLead);
      else qk_block(blk + 1, s, std::integral_constant<int, 2>{}, blk + kLead);
      if (restarts_left > 0 && flags_ask_restart(fl)) { restart = true; restarts_left--; break; }
      Sm st;
      float sc[8];
      unpack_scores(s, sc);
      pv_softmax(blk, std::true_type{}, std::true_type{}, sc, st, has_rows);
      if (has_rows) softmax_finish(blk + 1, sc, st);
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
    const bool e_row_ok = e_row < rows && e_rloc < kGrpRows && L > 0;
    // the row's four lanes combine their sums and their candidates for the dominant key
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);
    int top_tok = top_tag < 0 ? -1 : (top_tag >> 3) * kBlk + 16 * ((top_tag >> 2) & 1) + 4 * e_g + (top_tag & 3);
#pragma unroll
    for (int d = 16; d <= 32; d <<= 1) {
      const float op = __shfl_xor(top_p, d, 64);
      const int ot = __shfl_xor(top_tok, d, 64);
      const bool take = op > top_p || (op == top_p && ot >= 0 && (top_tok < 0 || ot < top_tok));
      top_p = take ? op : top_p;
      top_tok = take ? ot : top_tok;
    }
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    // Rows whose most probable key carries more than 1/16 of the weight leave a note for the merge kernel: the rounding
    // error of that key's probability (already divided by l) and the address of its latent vector in the cache.
    float corr = 0.f;
    KernArgPtr kp = cold();
    const __bf16* nope0 = kp->nope;
    const __bf16* vrow = nope0;
    // (the small forms carry every probability's rounding remainder through P.V themselves: nothing to add back)
    if (kRG == 4 && e_row_ok && top_tok >= 0 && top_p * 16.f > l_tot) {
      corr = (top_p - (float)(__bf16)top_p) * inv;
      if constexpr (kSparse) {
        int64_t slot = kp->sparse_rows[(int64_t)b * kp->sparse_stride + top_tok];
        slot = slot < 0 ? 0 : (slot > max_row ? max_row : slot);
        vrow = nope0 + slot * kp->nope_sr;
      } else {
        const int ctok = top_tok + ((kWindow && top_tok >= kp->win_sink) ? win_skip * kBlk : 0);   // position in the cache
        int page = ctok / kPage;
        const int mb = kp->max_blocks;
        page = page < mb ? page : mb - 1;
        int64_t pg = kp->block_table[(int64_t)b * kp->bt_stride + page];
        const int64_t np_ = kp->num_pages;
        pg = pg < 0 ? 0 : (pg >= np_ ? np_ - 1 : pg);
        vrow = nope0 + pg * kp->nope_sp + (int64_t)(ctok % kPage) * kp->nope_sr;
      }
    }
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

}  // namespace v3

template <bool kSparse, bool kWindow, int kRG, bool kWrite = false>
static int launch_form(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  const int rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<kSparse, kWindow, kRG, kWrite>, v3::kLdsB, "mla_decode_v3_kernel");
  if (rc != MLA_OK) return rc;
  hipLaunchKernelGGL((v3::mla_decode_v3_kernel<kSparse, kWindow, kRG, kWrite>), grid, dim3(512), v3::kLdsB, stream, p);
  return check_launch("mla_decode_v3_kernel");
}
constexpr int kNumCUs = 256;                               // MI355X
template <bool kSparse, bool kWindow, bool kWrite = false>
static int launch_rows(const DecodeParams& p, dim3 grid, hipStream_t stream) {
  // requests with at most 32 / 64 query rows (tokens x heads) take the forms that leave the missing rows out
  const int64_t r_max = (int64_t)p.max_q_len * p.num_heads;
  // (the form depends on the shape; all three get their LDS limit with the family's first launch, so that a later launch
  // under stream capture, where the limit cannot be raised, finds every form ready)
  {
    int rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<kSparse, kWindow, 1, kWrite>, v3::kLdsB, "mla_decode_v3_kernel");
    if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<kSparse, kWindow, 2, kWrite>, v3::kLdsB, "mla_decode_v3_kernel");
    if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<kSparse, kWindow, 4, kWrite>, v3::kLdsB, "mla_decode_v3_kernel");
    if (rc != MLA_OK) return rc;
  }
  if (r_max <= 32) return launch_form<kSparse, kWindow, 1, kWrite>(p, grid, stream);
  if (r_max <= 64) return launch_form<kSparse, kWindow, 2, kWrite>(p, grid, stream);
  // With few requests and short contexts (and with row lists, which are short by nature) the caller's chunks do not fill
  // the 256 CUs, and cutting the keys finer makes every workgroup pay a segment's start and end for a handful of blocks.
  // The rows are cut instead: groups of 64 or 32 rows, each with its own workgroup over the whole chunk (the groups of a
  // chunk sit next to each other on one XCD and share the cache rows in its L2).  Measured on row lists of 2048 keys,
  // 128 heads, eight chunks per token: 4 tokens 36.1 -> 26.9 us, 8 tokens 37.7 -> 28.8, 16 tokens 40.4 -> 33.3.
  {
    const int64_t wgs = (int64_t)grid.x * grid.z;
    if (wgs * 4 <= kNumCUs) { grid.z = (unsigned)((r_max + 31) / 32); return launch_form<kSparse, kWindow, 1, kWrite>(p, grid, stream); }
    if (wgs * 2 <= kNumCUs) { grid.z = (unsigned)((r_max + 63) / 64); return launch_form<kSparse, kWindow, 2, kWrite>(p, grid, stream); }
  }
  return launch_form<kSparse, kWindow, 4, kWrite>(p, grid, stream);
}

// Raises the dynamic-LDS limit of every dense form on the current device (what a launch does for its own form the first
// time it runs): a caller that will launch under stream capture, where that cannot be recorded, does it beforehand.
int prepare_decode_v3_dense_forms() {
  int rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<false, false, 1, false>, v3::kLdsB, "mla_decode_v3_kernel");
  if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<false, false, 2, false>, v3::kLdsB, "mla_decode_v3_kernel");
  if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)v3::mla_decode_v3_kernel<false, false, 4, false>, v3::kLdsB, "mla_decode_v3_kernel");
  return rc;
}

int launch_decode_v3(const DecodeParams& p, bool sparse, dim3 grid, hipStream_t stream) {
  if (sparse) return launch_rows<true, false>(p, grid, stream);
  if (p.win_skip) return launch_rows<false, true>(p, grid, stream);
  if (p.new_c) return launch_rows<false, false, true>(p, grid, stream);
  return launch_rows<false, false>(p, grid, stream);
}

}  // namespace mlahip
