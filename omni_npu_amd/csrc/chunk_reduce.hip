// N-way merge of the split-KV partials of the decode kernels (src/omni_npu/attention/ops.py:109-141 semantics): the second
// phase of mla_decode_bf16 / mla_decode_fp8 / dsa_sparse_decode_bf16 and the body of mla_splitkv_reduce.
#include "decode_params.hpp"
#include <type_traits>
#include <cstdlib>

namespace mlahip {

constexpr int kBlk = kPlanBlk;                             // tokens per block of the chunk plan
constexpr int kSegCost = kPlanSegCost;                     // start-up cost of a segment, in blocks

__device__ __forceinline__ int plan_num_blocks(int len) { return len > 0 ? (len + kBlk - 1) / kBlk : 0; }
__device__ __forceinline__ int plan_units(int len) { return len > 0 ? (len + kBlk - 1) / kBlk + kSegCost : 0; }
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

// N-way merge of the partials of the query rows (src/omni_npu/attention/ops.py:109-141), for the chunk layout written
// by the split kernels (decode_v3.hip, decode_v3_fp8.hip).  The partials of sequence b are those of the chunks that hold blocks of it, numbered
// chunk + b.  A wavefront merges kRedRows consecutive rows of one sequence (lane l owns columns 8l..8l+7): it derives
// the chunk list once, fetches the per-row records of up to kRedParts partials with scalar loads, then asks for the
// partials and the latent vectors of the flagged dominant keys together before it uses any of them - the kernel is a
// chain of dependent memory round trips, and this keeps the vector part of the chain at one.  (One row per wave keeps it
// at four waves per SIMD; the gathers of the dominant keys' vectors are a third of its time.)
// With many partials per sequence (few sequences, long contexts: up to 257 partials of one row) a single wavefront would
// walk them in dozens of dependent round trips, so the kWide form gives a row to a whole workgroup of kWideWaves wavefronts
// (eight while one workgroup per compute unit holds all rows, else four): wavefront w merges every kWideWaves-th partial,
// sixteen per pass, and the running states are merged through LDS at the end.
// With one chunk per sequence (large batches) a row has one partial, or two where a chunk border falls inside its
// sequence: the kFew form then gives a wavefront four rows of two partials, a quarter of the wavefronts and rounds.
// (four partials per pass in the one-wavefront form: 69 registers, seven wavefronts per SIMD, so the 8192 rows of the
// headline batch are resident in one round; a row with five or eight partials takes a second pass.  Eight per pass - 121
// registers, four wavefronts per SIMD, two rounds - measured 1 to 3 us slower per step on both shapes, five and six in
// between)
constexpr int kRedPartsNarrow = 4, kRedPartsWide = 16, kRedPartsFew = 2, kRedRowsFew = 4;
template <bool kWide, bool kFew, int kWideWaves = 4>
__global__ __launch_bounds__(kWide ? 64 * kWideWaves : 256) void mla_chunk_reduce_kernel(const ChunkReduceParams p) {
  constexpr int kRedParts = kWide ? kRedPartsWide : (kFew ? kRedPartsFew : kRedPartsNarrow);
  constexpr int kRedRows = kFew ? kRedRowsFew : 1;
  __shared__ float comb_ml[kWide ? 2 * kWideWaves : 1];            // wide: running maximum and sum of every wavefront
  __shared__ float comb_a[kWide ? kWideWaves * 64 * 8 : 1];        //       and their unnormalised rows
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int r_max = p.max_q_len * p.num_heads;
  const int groups = (r_max + kRedRows - 1) / kRedRows;     // row groups per sequence
  // (the wave number is made a scalar: everything derived from it, the addresses of the per-row records included, then
  // lives in scalar registers and is fetched with scalar loads)
  // Workgroups go to the eight XCDs round-robin in launch order; every XCD takes a contiguous eighth of the rows, as the split
  // kernels give every XCD a contiguous eighth of the chunks: a row's partials were written, and its neighbours' partials
  // are being read, through the same part of the memory system (headline merge 17.1 -> 16.0 us, row lists 53.8 -> 52.3 us
  // for split + merge).
  int64_t wg_id = blockIdx.x;
  if (!kWide && (gridDim.x & 7) == 0) wg_id = (int64_t)(blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int64_t gw_first = kWide ? (int64_t)blockIdx.x : wg_id * 4 + wave;
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
  const int mine = plan_units(p.seq_lens[b]);
  int tot_units = 0, before = 0;
  for (int i = lane; i < p.batch; i += 64) {
    const int c = plan_units(p.seq_lens[i]);
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
    // wide: wavefront w takes the chunks c + w, c + w + 8, ...; where chunks have to be tested one by one (tiny
    // workloads, a handful of partials) wavefront 0 takes them all
    int c_step = 1;
    if constexpr (kWide) {
      if (dense_chunks) { c += wave; c_step = kWideWaves; }
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
      for (int w = 0; w < kWideWaves; w++) mm = fmaxf(mm, comb_ml[w * 2]);
      float tt = 0.f, aa[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < kWideWaves; w++) {
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
  // many partials: past a dozen per row the wide form wins, as long as all rows' workgroups are resident at once (two
  // per CU at its register use)
  const bool wide = per_seq > 12 && (int64_t)p.batch * r_max <= 512;
  // one or two partials and rows for more than one round of resident wavefronts: four rows per wavefront
  const bool few = !wide && per_seq <= kRedPartsFew && (int64_t)p.batch * r_max > 16384;
  if (wide) {
    const int64_t row_groups = (int64_t)p.batch * r_max;
    const int64_t wgs = row_groups < (1ll << 30) ? row_groups : (1ll << 30);
    // (measured, 128 heads: one sequence of 128k keys 25.5 -> 18.8 us with eight wavefronts per row; four sequences, i.e. two
    // rounds of such workgroups, 16.0 us with four wavefronts against 19.2 with eight)
    if (row_groups <= 256) hipLaunchKernelGGL((mla_chunk_reduce_kernel<true, false, 8>), dim3((unsigned)wgs), dim3(512), 0, stream, p);
    else hipLaunchKernelGGL((mla_chunk_reduce_kernel<true, false, 4>), dim3((unsigned)wgs), dim3(256), 0, stream, p);
  } else if (few) {
    const int64_t row_groups = (int64_t)p.batch * ((r_max + kRedRowsFew - 1) / kRedRowsFew);
    hipLaunchKernelGGL((mla_chunk_reduce_kernel<false, true>), dim3((unsigned)((row_groups + 3) / 4)), dim3(256), 0, stream, p);
  } else {
    const int64_t row_groups = (int64_t)p.batch * r_max;
    hipLaunchKernelGGL((mla_chunk_reduce_kernel<false, false>), dim3((unsigned)((row_groups + 3) / 4)), dim3(256), 0, stream, p);
  }
  return check_launch("mla_chunk_reduce_kernel");
}

}  // namespace mlahip
