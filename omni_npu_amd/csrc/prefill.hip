// Non-absorbed varlen MLA attention for prefill (suffix, causal) and for chunked-context chunks (no mask),
// with log-sum-exp output.
//
// Replaces the prefill calls of torch.ops.npu.npu_fused_infer_attention_score in
// src/omni_npu/attention/backends/mla.py:574-590 (suffix: input_layout "TND", sparse_mode 3, optional LSE) and
// :415-431 (context chunk: no mask, LSE): per sequence b, head n, query i
//   s_j = scale * (q_nope[i,n] . k_nope[j,n] + q_pe[i,n] . k_pe[j]),   j <= i + (sk - sq) when causal
//   o   = sum_j softmax(s)_j v[j,n],   lse = log sum_j exp(s_j)          (k_pe is shared by all heads, mla.py:579)
//
// One workgroup = 4 wavefronts = (128 query rows, one head, one sequence); each wavefront owns 32 rows with its
// 192-wide query in registers (B operand of S^T = K Q^T) and a 128 x 32 fp32 accumulator O^T.  Key tiles of 64 keys
// (nope 64 x 256 B, rope 64 x 128 B, V 64 x 256 B) are copied global -> LDS without touching registers, double
// buffered; V^T operands come from transposed LDS reads, so P^T stays in registers exactly as in the decode kernel.
//
// P.V runs on fp16: the V part of a landed tile is converted from bf16 to fp16 where it lies (same size, same swizzle:
// element by element), once for the four wavefronts, and the probabilities are rounded to fp16, so they keep 11
// significant bits instead of bf16's 8.  (With bf16 probabilities AND a bf16 result, flat attention over values
// unrelated to the keys lands at 2.2e-3 of mean relative error whatever else a kernel does: each rounding alone is
// 1.4e-3 to 1.7e-3.)  The conversion is exact for |v| in [2^-14, 65504]; smaller values lose at most 2^-25 absolute,
// larger ones saturate (round toward zero never makes an infinity).
#include "mla_common.hpp"

namespace mlahip {

constexpr int kPfTile = 64;
constexpr int kPfKnB = kPfTile * 256;            // 16384  k_nope tile
constexpr int kPfKrB = kPfTile * 128;            // 8192   k_pe tile
constexpr int kPfVB = kPfTile * 256;             // 16384  v tile
constexpr int kPfBufB = kPfKnB + kPfKrB + kPfVB; // 40960
constexpr int kPfLdsB = 2 * kPfBufB;             // 81920
constexpr int kPfRows = 128;

__device__ __forceinline__ int pf_swz16(int r) {  // bijection of r % 16, also spreads 4 consecutive rows x 64 B
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r1 ^ r3) << 3) | (r0 << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int pf_swz8(int r) {
  int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r0 ^ r3) << 2) | (r1 << 1) | r2;
}

struct PrefillParams {
  const __bf16* q_nope; int64_t qn_st, qn_sh;
  const __bf16* q_pe; int64_t qp_st, qp_sh;
  const __bf16* k_nope; int64_t kn_st, kn_sh;
  const __bf16* k_pe; int64_t kp_st;
  const __bf16* v; int64_t v_st, v_sh;
  const int32_t* cu_q; const int32_t* cu_k;
  int32_t batch, num_heads, causal;
  int32_t window;                                            // keep only the newest `window` visible keys of a row; 0 = all
  float scale_log2;
  void* out; int64_t o_st, o_sh; int32_t out_fp32;
  float* lse; // [T, N]
  // optional state to continue from: the normalised result and log-sum-exp of an attention over OTHER keys of the same rows
  // (an earlier context chunk); the launch then returns the attention over the union, as a merge of the two would
  const float* prev_out; int64_t po_st, po_sh;
  const float* prev_lse;  // [T, N]
};

// copy one 64-key tile (keys k0 .. k0+63 of the flat key axis, clamped to klast) of head `head`
__device__ __forceinline__ void pf_issue_tile(const PrefillParams& p, int64_t k0, int64_t klast, int head, uint32_t buf,
                                              int wave, int lane) {
  // k_nope and v: 16 granules per row, one wave instruction covers 4 rows; 16 instructions per tensor, 4 per wave
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = (wave * 4 + i) * 4 + (lane >> 4);
    int64_t key = k0 + r;
    key = key < klast ? key : klast;
    const int c = (lane & 15) ^ pf_swz16(r & 15);
    dma16_v(p.k_nope + key * p.kn_st + (int64_t)head * p.kn_sh + c * 8, buf + (wave * 4 + i) * 1024);
    dma16_v(p.v + key * p.v_st + (int64_t)head * p.v_sh + c * 8, buf + kPfKnB + kPfKrB + (wave * 4 + i) * 1024);
  }
  // k_pe: 8 granules per row, one wave instruction covers 8 rows; 8 instructions, 2 per wave
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = (wave * 2 + i) * 8 + (lane >> 3);
    int64_t key = k0 + r;
    key = key < klast ? key : klast;
    const int c = (lane & 7) ^ pf_swz8(r & 15);
    dma16_v(p.k_pe + key * p.kp_st + c * 8, buf + kPfKnB + (wave * 2 + i) * 1024);
  }
}

// Per-lane source offsets of a FULL tile (all 64 keys exist), relative to the tile's first key: the copies then need one
// uniform base per tensor and no per-lane address arithmetic.
struct PfLaneOffsets { uint32_t kn[4], v[4], kp[2]; };
__device__ __forceinline__ PfLaneOffsets pf_lane_offsets(const PrefillParams& p, int wave, int lane) {
  PfLaneOffsets o;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = (wave * 4 + i) * 4 + (lane >> 4);
    const int c = (lane & 15) ^ pf_swz16(r & 15);
    o.kn[i] = (uint32_t)(r * p.kn_st * 2 + c * 16);
    o.v[i] = (uint32_t)(r * p.v_st * 2 + c * 16);
  }
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = (wave * 2 + i) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ pf_swz8(r & 15);
    o.kp[i] = (uint32_t)(r * p.kp_st * 2 + c * 16);
  }
  return o;
}
__device__ __forceinline__ void pf_issue_full_tile(const PrefillParams& p, const PfLaneOffsets& o, int64_t k0, int head,
                                                   uint32_t buf, int wave) {
  const char* kn = (const char*)(p.k_nope + k0 * p.kn_st + (int64_t)head * p.kn_sh);
  const char* vv = (const char*)(p.v + k0 * p.v_st + (int64_t)head * p.v_sh);
  const char* kp = (const char*)(p.k_pe + k0 * p.kp_st);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    dma16_sv(kn, o.kn[i], buf + (wave * 4 + i) * 1024);
    dma16_sv(vv, o.v[i], buf + kPfKnB + kPfKrB + (wave * 4 + i) * 1024);
  }
#pragma unroll
  for (int i = 0; i < 2; i++) dma16_sv(kp, o.kp[i], buf + kPfKnB + (wave * 2 + i) * 1024);
}

// kHalf: k_nope, k_pe and v hold fp16 instead of bf16 (a caller that makes them with an fp16 GEMM): both products run on
// fp16 (the query is converted once, in registers) and no tile is converted.
template <bool kHalf>
__global__ __launch_bounds__(256, 2) void mla_prefill_varlen_kernel(const PrefillParams p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h32 = lane & 31, half = lane >> 5;
  // Workgroups go to the eight XCDs round-robin in launch order (x fastest), and each XCD has its own L2.  All query
  // blocks of one (sequence, head) stream the same keys and values, so they are renumbered to sit on ONE XCD, next to each
  // other in its queue: they then run at the same time and all but the first find the K / V tiles in that L2.
  int qb = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
  {
    const int nqb = gridDim.x, npairs = gridDim.y * gridDim.z;
    if ((npairs & 7) == 0) {
      const int lin = blockIdx.x + nqb * (blockIdx.y + gridDim.y * blockIdx.z);
      const int j = lin >> 3, pair = (j / nqb) * 8 + (lin & 7);
      qb = j % nqb;
      head = pair % gridDim.y;
      b = pair / gridDim.y;
    }
  }
  const int q0 = p.cu_q[b], sq = p.cu_q[b + 1] - q0;
  const int k0 = p.cu_k[b], sk = p.cu_k[b + 1] - k0;
  if (qb * kPfRows >= sq) return;

  const int row = qb * kPfRows + wave * 32 + h32;            // query index inside the sequence
  const bool row_ok = row < sq;
  const int shift = sk - sq;                                  // right-down alignment of the causal mask
  int limit = p.causal ? row + shift + 1 : sk;                // visible keys of this row
  limit = !row_ok ? 0 : (limit < 0 ? 0 : (limit > sk ? sk : limit));
  int wave_min_limit = limit;                                 // fewest keys any row of this wave can see
  int wave_max_limit = limit;                                 // most keys any row of this wave can see
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int other = __shfl_xor(wave_min_limit, o, 64); wave_min_limit = other < wave_min_limit ? other : wave_min_limit;
    const int more = __shfl_xor(wave_max_limit, o, 64); wave_max_limit = more > wave_max_limit ? more : wave_max_limit;
  }
  wave_min_limit = __builtin_amdgcn_readfirstlane(wave_min_limit);
  wave_max_limit = __builtin_amdgcn_readfirstlane(wave_max_limit);
  // Sliding window: a row sees keys [lo, limit).  lo grows with the row, so the first row of the workgroup gives the
  // first key any row needs, and the largest lo of a wave tells which blocks need the mask at their front.
  const int lo = (p.window > 0 && limit > p.window) ? limit - p.window : 0;
  int wave_max_lo = lo;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) { const int other = __shfl_xor(wave_max_lo, o, 64); wave_max_lo = other > wave_max_lo ? other : wave_max_lo; }
  wave_max_lo = __builtin_amdgcn_readfirstlane(wave_max_lo);
  int wg_lo = 0;
  if (p.window > 0) {
    int lim0 = p.causal ? qb * kPfRows + shift + 1 : sk;
    lim0 = lim0 < 0 ? 0 : (lim0 > sk ? sk : lim0);
    wg_lo = lim0 > p.window ? lim0 - p.window : 0;
  }
  const int first_tile = wg_lo / kPfTile;
  // keys any row of this workgroup can see
  int wg_limit = sk;
  if (p.causal) {
    int last_row = qb * kPfRows + kPfRows - 1;
    last_row = last_row < sq - 1 ? last_row : sq - 1;
    wg_limit = last_row + shift + 1;
    wg_limit = wg_limit < 0 ? 0 : (wg_limit > sk ? sk : wg_limit);
  }
  const int tiles = (wg_limit + kPfTile - 1) / kPfTile;

  const int64_t tq = q0 + (row_ok ? row : 0);
  f32x16 acc[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  if (p.prev_out != nullptr && row_ok) {
    // Continue from (out, lse) over other keys: running maximum = lse (as a base-2 exponent), running sum = 1, accumulator
    // = out.  A row without earlier keys comes with lse = -inf (+inf is read the same way, as the two-way merge does) and
    // starts empty.  The sum lives in the row's lower half-wave lane; the halves are added at the end.
    const float lse_prev = p.prev_lse[tq * p.num_heads + head];
    if (lse_prev != INFINITY && lse_prev != -INFINITY) {
      m_run = lse_prev * kLog2e;
      l_run = half == 0 ? 1.f : 0.f;
      const float* po = p.prev_out + tq * p.po_st + (int64_t)head * p.po_sh + 4 * half;
#pragma unroll
      for (int db = 0; db < 4; db++)
#pragma unroll
        for (int rg = 0; rg < 4; rg++) {
          const f32x4 v = *(const f32x4*)(po + db * 32 + rg * 8);
#pragma unroll
          for (int e = 0; e < 4; e++) acc[db][rg * 4 + e] = v[e];
        }
    }
  }

  if (tiles > 0) {
    const uint32_t lds0 = lds_addr_of(lds);
    const int64_t klast = (int64_t)k0 + sk - 1;
    const PfLaneOffsets lane_off = pf_lane_offsets(p, wave, lane);
    const bool fast_ok = (uint64_t)p.kn_st * 128 < (1u << 31) && (uint64_t)p.v_st * 128 < (1u << 31) && (uint64_t)p.kp_st * 128 < (1u << 31);
    auto issue = [&](int tile, uint32_t buf) {
      const int64_t first = (int64_t)k0 + (int64_t)tile * kPfTile;
      if (fast_ok && first + kPfTile - 1 <= klast) pf_issue_full_tile(p, lane_off, first, head, buf, wave);
      else pf_issue_tile(p, first, klast, head, buf, wave, lane);
    };
    issue(first_tile, lds0 + (first_tile & 1) * kPfBufB);

    bf16x8 qf[12];
    {
      const __bf16* qn = p.q_nope + tq * p.qn_st + (int64_t)head * p.qn_sh + half * 8;
      const __bf16* qp = p.q_pe + tq * p.qp_st + (int64_t)head * p.qp_sh + half * 8;
      const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int kk = 0; kk < 8; kk++) { bf16x8 v = *(const bf16x8*)(qn + kk * 16); qf[kk] = row_ok ? v : zero; }
#pragma unroll
      for (int kk = 0; kk < 4; kk++) { bf16x8 v = *(const bf16x8*)(qp + kk * 16); qf[8 + kk] = row_ok ? v : zero; }
      if constexpr (kHalf) {
#pragma unroll
        for (int kk = 0; kk < 12; kk++) {
          f16x8 h;
#pragma unroll
          for (int e = 0; e < 8; e++) h[e] = (_Float16)(float)qf[kk][e];
          qf[kk] = __builtin_bit_cast(bf16x8, h);
        }
      }
    }
    // per-lane LDS offsets
    const int fk = pf_swz16(h32 & 15), fr = pf_swz8(h32 & 15);
    int koff[8], roff[4];
#pragma unroll
    for (int j = 0; j < 8; j++) koff[j] = h32 * 256 + (((j * 2 + half) ^ fk) << 4);
#pragma unroll
    for (int j = 0; j < 4; j++) roff[j] = kPfKnB + h32 * 128 + (((j * 2 + half) ^ fr) << 4);
    const int g16 = lane >> 4, j16 = lane & 15;
    const int v_row = 4 * (g16 >> 1) + (j16 >> 2);
    const int v_cl = 2 * (g16 & 1) + ((j16 & 3) >> 1);
    const int v_in = (j16 & 1) * 8;
    int voff[2][4];                                           // [rd][db]
#pragma unroll
    for (int rd = 0; rd < 2; rd++) {
      const int rr = v_row + 8 * rd;
      const int f = pf_swz16(rr & 15);
#pragma unroll
      for (int db = 0; db < 4; db++) voff[rd][db] = kPfKnB + kPfKrB + rr * 256 + v_in + (((db * 4 + v_cl) ^ f) << 4);
    }

    for (int tile = first_tile; tile < tiles; tile++) {
      char* buf = lds + (tile & 1) * kPfBufB;
      // this tile has landed (only its copies are in flight here) and everyone is done with the other buffer
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      if (tile + 1 < tiles) issue(tile + 1, lds0 + ((tile + 1) & 1) * kPfBufB);
      const int key_base = tile * kPfTile;
      // V of this tile goes from bf16 to fp16 where it lies (thread t takes the 16-byte pieces t, t + 256, ...), then a
      // barrier: the four wavefronts read each other's pieces.  (Tried: the conversion's arithmetic and writes behind the
      // first block's score MFMAs, and the next tile converted between the two blocks of this one - both slower.)
      char* vt = buf + kPfKnB + kPfKrB + (int)threadIdx.x * 16;
      if constexpr (!kHalf) {
        u32x4 w[4];
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = *(const u32x4*)(vt + i * 4096);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float f_lo = __builtin_bit_cast(float, w[i][e] << 16);
            const float f_hi = __builtin_bit_cast(float, w[i][e] & 0xffff0000u);
            w[i][e] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(f_lo, f_hi));
          }
#pragma unroll
        for (int i = 0; i < 4; i++) *(u32x4*)(vt + i * 4096) = w[i];
        lds_barrier();
      }
#pragma unroll 1
      for (int tb = 0; tb < 2; tb++) {
        const bool active = key_base + tb * 32 < wave_max_limit && key_base + tb * 32 + 32 > wg_lo;
        if (!active) continue;
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
          bf16x8 a = *(const bf16x8*)(buf + tb * 32 * 256 + koff[kk]);
          if constexpr (kHalf) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, qf[kk]), s, 0, 0, 0);
          else s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[kk], s, 0, 0, 0);
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
          bf16x8 a = *(const bf16x8*)(buf + tb * 32 * 128 + roff[kk]);
          if constexpr (kHalf) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, qf[8 + kk]), s, 0, 0, 0);
          else s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[8 + kk], s, 0, 0, 0);
        }
        // Only blocks that some row of this wave cannot see in full pay for the mask (causal diagonal, end of the keys,
        // rows past the end of the sequence); everywhere else the scores go straight to the maximum.  The scale is
        // folded into the exponent's multiply-add (scale > 0, so the maximum of the raw scores is the raw maximum).
        if (key_base + tb * 32 + 32 > wave_min_limit || key_base + tb * 32 < wave_max_lo) {
          const int key_lane0 = key_base + tb * 32 + 4 * half;
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = key_lane0 + 8 * (r >> 2) + (r & 3);
            s[r] = (key < limit && key >= lo) ? s[r] : -INFINITY;
          }
        }
        float mx = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
        for (int r = 3; r < 15; r += 2) mx = fmaxf(fmaxf(mx, s[r]), s[r + 1]);
        mx = fmaxf(mx, s[15]);
        mx = fmaxf(mx, xor32(mx)) * p.scale_log2;
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = fast_exp2(m_run - m_safe);
        const float neg = -m_safe;
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
          s[r] = fast_exp2(__builtin_fmaf(s[r], p.scale_log2, neg));
          psum += s[r];
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
          for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][r] *= alpha;
        }
        f16x8 pb[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
          for (int e = 0; e < 8; e++) pb[kb][e] = (_Float16)s[kb * 8 + e];
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
          for (int kb = 0; kb < 2; kb++) {
            bf16x4 lo = lds_read_tr16(buf + (tb * 32 + kb * 16) * 256 + voff[0][db]);
            bf16x4 hi = lds_read_tr16(buf + (tb * 32 + kb * 16) * 256 + voff[1][db]);
            bf16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), pb[kb], acc[db], 0, 0, 0);
          }
      }
    }
  }

  const float l_tot = l_run + xor32(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (row_ok) {
    if (p.lse && half == 0) p.lse[tq * p.num_heads + head] = l_tot > 0.f ? (m_run + fast_log2(l_tot)) * kLn2 : -INFINITY;
    const int64_t o = tq * p.o_st + (int64_t)head * p.o_sh + 4 * half;
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
      for (int rg = 0; rg < 4; rg++) {
        const int d = db * 32 + rg * 8;
        if (p.out_fp32) {
          f32x4 v = {acc[db][rg * 4] * inv, acc[db][rg * 4 + 1] * inv, acc[db][rg * 4 + 2] * inv, acc[db][rg * 4 + 3] * inv};
          *(f32x4*)((float*)p.out + o + d) = v;
        } else {
          bf16x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = (__bf16)(acc[db][rg * 4 + e] * inv);
          *(bf16x4*)((__bf16*)p.out + o + d) = v;
        }
      }
  }
}

}  // namespace mlahip
using namespace mlahip;

// out_dtype: 0 = bf16, 1 = fp32; window: 0 = every visible key, w = the newest w of them.  q_nope [T,N,128], q_pe [T,N,64], k_nope [Tk,N,128], k_pe [Tk,64], v [Tk,N,128].
static int prefill_varlen_impl(const char* what, const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_pe,
                               int64_t qp_stride_t, int64_t qp_stride_h, const void* k_nope, int64_t kn_stride_t,
                               int64_t kn_stride_h, const void* k_pe, int64_t kp_stride_t, const void* v,
                               int64_t v_stride_t, int64_t v_stride_h, const int32_t* cu_q, const int32_t* cu_k,
                               int32_t batch, int32_t num_heads, int32_t max_q_len, int32_t causal, int32_t window,
                               float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, int32_t out_dtype,
                               float* lse_out, const float* prev_out, int64_t prev_stride_t, int64_t prev_stride_h,
                               const float* prev_lse, hipStream_t stream) {
  MLA_REQUIRE(q_nope && q_pe && k_nope && k_pe && v && cu_q && cu_k && out, MLA_ERR_NULL, "%s: null pointer argument", what);
  MLA_REQUIRE(batch >= 0 && num_heads >= 1 && max_q_len >= 0 && batch <= 65535 && num_heads <= 65535 && window >= 0,
              MLA_ERR_SHAPE, "%s: batch=%d num_heads=%d max_q_len=%d window=%d", what, batch, num_heads, max_q_len, window);
  const bool kv_half = (out_dtype & 16) != 0;              // k_nope, k_pe and v hold fp16 (MLA_PREFILL_KV_F16)
  out_dtype &= ~16;
  MLA_REQUIRE(out_dtype == 0 || out_dtype == 1, MLA_ERR_UNSUPPORTED, "%s: out dtype code %d", what, out_dtype);
  MLA_REQUIRE(scale > 0.f, MLA_ERR_UNSUPPORTED, "%s: the softmax scale must be positive (got %g)", what, (double)scale);
  MLA_REQUIRE(qn_stride_t % 8 == 0 && qn_stride_h % 8 == 0 && qp_stride_t % 8 == 0 && qp_stride_h % 8 == 0 &&
                  kn_stride_t % 8 == 0 && kn_stride_h % 8 == 0 && kp_stride_t % 8 == 0 && v_stride_t % 8 == 0 &&
                  v_stride_h % 8 == 0 && out_stride_t % 4 == 0 && out_stride_h % 4 == 0 && (uintptr_t)q_nope % 16 == 0 &&
                  (uintptr_t)q_pe % 16 == 0 && (uintptr_t)k_nope % 16 == 0 && (uintptr_t)k_pe % 16 == 0 &&
                  (uintptr_t)v % 16 == 0 && (uintptr_t)out % 16 == 0,
              MLA_ERR_SHAPE, "%s: rows must be 16-byte aligned", what);
  MLA_REQUIRE((prev_out == nullptr) == (prev_lse == nullptr), MLA_ERR_NULL, "%s: the earlier result and its log-sum-exp go together", what);
  MLA_REQUIRE(prev_out == nullptr || (prev_stride_t % 4 == 0 && prev_stride_h % 4 == 0 && (uintptr_t)prev_out % 16 == 0),
              MLA_ERR_SHAPE, "%s: rows of the earlier result must be 16-byte aligned", what);
  if (batch == 0 || max_q_len == 0) return MLA_OK;
  PrefillParams p;
  p.q_nope = (const __bf16*)q_nope; p.qn_st = qn_stride_t; p.qn_sh = qn_stride_h;
  p.q_pe = (const __bf16*)q_pe; p.qp_st = qp_stride_t; p.qp_sh = qp_stride_h;
  p.k_nope = (const __bf16*)k_nope; p.kn_st = kn_stride_t; p.kn_sh = kn_stride_h;
  p.k_pe = (const __bf16*)k_pe; p.kp_st = kp_stride_t;
  p.v = (const __bf16*)v; p.v_st = v_stride_t; p.v_sh = v_stride_h;
  p.cu_q = cu_q; p.cu_k = cu_k; p.batch = batch; p.num_heads = num_heads; p.causal = causal; p.window = window;
  p.scale_log2 = scale * kLog2e;
  p.out = out; p.o_st = out_stride_t; p.o_sh = out_stride_h; p.out_fp32 = out_dtype;
  p.lse = lse_out;
  p.prev_out = prev_out; p.po_st = prev_stride_t; p.po_sh = prev_stride_h; p.prev_lse = prev_lse;
  int rc = ensure_dynamic_lds((const void*)mla_prefill_varlen_kernel<false>, kPfLdsB, what);
  if (rc == MLA_OK) rc = ensure_dynamic_lds((const void*)mla_prefill_varlen_kernel<true>, kPfLdsB, what);
  if (rc != MLA_OK) return rc;
  dim3 grid((max_q_len + kPfRows - 1) / kPfRows, num_heads, batch);
  if (kv_half) hipLaunchKernelGGL(mla_prefill_varlen_kernel<true>, grid, dim3(256), kPfLdsB, stream, p);
  else hipLaunchKernelGGL(mla_prefill_varlen_kernel<false>, grid, dim3(256), kPfLdsB, stream, p);
  return check_launch("mla_prefill_varlen_kernel");
}

extern "C" int mla_prefill_varlen(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_pe,
                                  int64_t qp_stride_t, int64_t qp_stride_h, const void* k_nope, int64_t kn_stride_t,
                                  int64_t kn_stride_h, const void* k_pe, int64_t kp_stride_t, const void* v,
                                  int64_t v_stride_t, int64_t v_stride_h, const int32_t* cu_q, const int32_t* cu_k,
                                  int32_t batch, int32_t num_heads, int32_t max_q_len, int32_t causal, int32_t window,
                                  float scale, void* out, int64_t out_stride_t, int64_t out_stride_h, int32_t out_dtype,
                                  float* lse_out, hipStream_t stream) {
  return prefill_varlen_impl("mla_prefill_varlen", q_nope, qn_stride_t, qn_stride_h, q_pe, qp_stride_t, qp_stride_h, k_nope,
                             kn_stride_t, kn_stride_h, k_pe, kp_stride_t, v, v_stride_t, v_stride_h, cu_q, cu_k, batch,
                             num_heads, max_q_len, causal, window, scale, out, out_stride_t, out_stride_h, out_dtype, lse_out,
                             nullptr, 0, 0, nullptr, stream);
}

// The same attention continued from an earlier result over other keys of the same rows (prev_out fp32 [T,N,128] with its
// strides, prev_lse fp32 [T,N] contiguous): what the attention followed by the two-way merge returns, in one launch.
// out may be prev_out and lse_out may be prev_lse (every row reads its own state before it writes it).
extern "C" int mla_prefill_varlen_continue(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_pe,
                                           int64_t qp_stride_t, int64_t qp_stride_h, const void* k_nope, int64_t kn_stride_t,
                                           int64_t kn_stride_h, const void* k_pe, int64_t kp_stride_t, const void* v,
                                           int64_t v_stride_t, int64_t v_stride_h, const int32_t* cu_q, const int32_t* cu_k,
                                           int32_t batch, int32_t num_heads, int32_t max_q_len, int32_t causal, int32_t window,
                                           float scale, void* out, int64_t out_stride_t, int64_t out_stride_h,
                                           int32_t out_dtype, float* lse_out, const float* prev_out, int64_t prev_stride_t,
                                           int64_t prev_stride_h, const float* prev_lse, hipStream_t stream) {
  MLA_REQUIRE(prev_out && prev_lse, MLA_ERR_NULL, "mla_prefill_varlen_continue: null pointer argument");
  return prefill_varlen_impl("mla_prefill_varlen_continue", q_nope, qn_stride_t, qn_stride_h, q_pe, qp_stride_t, qp_stride_h,
                             k_nope, kn_stride_t, kn_stride_h, k_pe, kp_stride_t, v, v_stride_t, v_stride_h, cu_q, cu_k, batch,
                             num_heads, max_q_len, causal, window, scale, out, out_stride_t, out_stride_h, out_dtype, lse_out,
                             prev_out, prev_stride_t, prev_stride_h, prev_lse, stream);
}
