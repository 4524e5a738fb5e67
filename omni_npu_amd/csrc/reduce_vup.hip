// Merge of the split-KV partials fused with the value up-projection (C-ABI entry mla_splitkv_reduce_vup).
//
// Replaces, for the decode tokens, the N-way merge of src/omni_npu/attention/ops.py:109-141 followed by the
// reference's _v_up_proj (src/omni_npu/attention/backends/mla.py:309-315; DSA: dsa.py:233-240):
//   o[t,n,:]   = merge over the partials of (t, n)                         (fp32, rounded to bf16 as the unfused path does)
//   out[t, n*V + v] = sum_c o[t,n,c] * W_UV[n,c,v]                         (bf16 MFMA, fp32 accumulation), V = 128
// The unfused path writes o [N,T,512], runs a batched GEMM into [N,T,V], transposes that into [T, N*V] and copies it
// into the caller's output: four launches and three round trips through memory for 2 MB of result.
//
// One workgroup = one head and a run of tokens.  Its 16 wavefronts first ask for the head's W_UV (512 x 128 bf16 =
// 128 KiB) as global -> LDS copies, then each merges the partials of ONE token's row (the copies land underneath),
// writes the bf16 row into a 16-row LDS tile, and four wavefronts multiply the tile with W_UV out of LDS: W^T is the
// first MFMA operand (32 output columns per wavefront), read with transposed LDS reads exactly like V^T in the decode
// kernel, the merged rows are the second operand, so a lane ends up with four consecutive output columns of one token.
#include "mla_common.hpp"
#include "decode_params.hpp"

namespace mlahip {
namespace {

constexpr int kVupTok = 16;                     // tokens per pass: one per wavefront
constexpr int kVupV = 128;                      // v_head_dim
constexpr int kVupWB = kDNope * kVupV * 2;      // 131072: W_UV of one head, row c at c * 256
constexpr int kVupOB = kVupTok * kDNope * 2;    // 16384: merged rows of one pass, 1 KiB each
constexpr int kVupFlagOff = kVupWB + kVupOB;    // one int per token of the pass: its row is valid
constexpr int kVupLdsB = kVupFlagOff + 64;
constexpr int kVupParts = 6;                    // partials of a row asked for together
constexpr int kVupAhead = 4;                    // GEMM steps whose operands are requested ahead (at most 4: the wait ladder)

__device__ __forceinline__ int vup_wave_sum(int v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}

// Merge of the partials of row `row` of sequence b (all arguments wave-uniform), lane l owning columns 8l .. 8l+7.
// Same bookkeeping as mla_chunk_reduce_kernel: the partials of a sequence are those of the chunks that hold blocks of
// it, numbered chunk + b; with at least one work unit per chunk they are the consecutive numbers between the two the
// split kernel left in seg_ids, otherwise the chunk boundaries are worked out from the sequence lengths.
__device__ __forceinline__ void vup_merge_row(const ChunkReduceParams& p, int b, int row, int lane, float& m, float& tot,
                                              float (&a)[8]) {
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  const int r_max = p.max_q_len * p.num_heads;
  const int id_first = p.seg_ids[2 * b], id_last = p.seg_ids[2 * b + 1];
  const int mine = plan_work_units(p.seq_lens[b]);
  int tot_units = 0, before = 0;
  for (int i = lane; i < p.batch; i += 64) {
    const int c = plan_work_units(p.seq_lens[i]);
    tot_units += c;
    before += i < b ? c : 0;
  }
  tot_units = __builtin_amdgcn_readfirstlane(vup_wave_sum(tot_units));
  before = __builtin_amdgcn_readfirstlane(vup_wave_sum(before));
  if (mine <= 0) return;
  const int64_t G = p.num_chunks, T = tot_units;
  auto holds_blocks = [&](int64_t c) -> bool {
    const int64_t cb = c * T / G, ce = (c + 1) * T / G;
    const int64_t lo = cb > before ? cb : before, hi = ce < before + mine ? ce : before + mine;
    int64_t rlo = lo - before - kPlanSegCost, rhi = hi - before - kPlanSegCost;
    rlo = rlo < 0 ? 0 : rlo;
    rhi = rhi < 0 ? 0 : rhi;
    return rhi > rlo;
  };
  const bool dense_chunks = T >= G;
  int c, c_last;
  if (dense_chunks) {
    c = id_first - b;
    c_last = id_last - b;
  } else {
    c = (int)((((int64_t)before + 1) * G - 1) / T);
    c_last = (int)((((int64_t)before + mine) * G - 1) / T);
  }
  while (c <= c_last) {
    int64_t part[kVupParts];
    int np = 0;
#pragma unroll
    for (int q = 0; q < kVupParts; q++) {
      while (c <= c_last && !dense_chunks && !holds_blocks(c)) c++;
      part[q] = c <= c_last ? (int64_t)(c + b) * r_max + row : 0;
      if (c <= c_last) { np++; c++; }
    }
    // records by scalar loads (uniform addresses), then the partials and the latent vectors of the flagged dominant
    // keys in one vector round trip
    float lse[kVupParts], cs[kVupParts];
    const __bf16* cp[kVupParts];
#pragma unroll
    for (int q = 0; q < kVupParts; q++) {
      const bool on = q < np;
      lse[q] = on ? p.lse_part[part[q]] : -INFINITY;
      cs[q] = on ? p.corr_scale[part[q]] : 0.f;
      cp[q] = p.corr_row[part[q]];
      if (lse[q] == INFINITY || lse[q] == -INFINITY) cs[q] = 0.f;
    }
    h8 v[kVupParts];
    bf16x8 kv[kVupParts];
#pragma unroll
    for (int q = 0; q < kVupParts; q++) {
      v[q] = *(const h8*)(p.o_part + part[q] * kDNope + lane * 8);
      if (cs[q] != 0.f) kv[q] = *(const bf16x8*)(cp[q] + lane * 8);
    }
#pragma unroll
    for (int q = 0; q < kVupParts; q++) {
      const float l = lse[q];
      if (l == INFINITY || l == -INFINITY) continue;
      const float mn = fmaxf(m, l);
      const float so = __expf(m - mn), w = __expf(l - mn);
      m = mn;
      tot = tot * so + w;
#pragma unroll
      for (int e = 0; e < 8; e++) a[e] = a[e] * so + (float)v[q][e] * w;
      if (cs[q] != 0.f) {
#pragma unroll
        for (int e = 0; e < 8; e++) a[e] += (float)kv[q][e] * (w * cs[q]);
      }
    }
  }
}

}  // namespace

struct ReduceVupParams {
  ChunkReduceParams r;                 // r.out: [T, N * 128] through (out_st, out_sh)
  const __bf16* w_uv; int64_t w_sn, w_sk;   // W_UV [N, 512, 128]: head stride, row stride (elements)
  int32_t num_tokens, passes;          // a workgroup handles passes * 16 consecutive tokens
};

__global__ __launch_bounds__(1024) void mla_reduce_vup_kernel(const ReduceVupParams pp) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const ChunkReduceParams& p = pp.r;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  // Workgroups go to the eight XCDs round-robin in launch order (x fastest) and each XCD has its own L2: the token
  // blocks of one head read the same 128 KiB of W_UV, so they are renumbered to sit on one XCD, next to each other.
  int tb = blockIdx.x, head = blockIdx.y;
  if ((gridDim.y & 7) == 0) {
    const int lin = blockIdx.x + gridDim.x * blockIdx.y;
    const int j = lin >> 3;
    tb = j % gridDim.x;
    head = (j / gridDim.x) * 8 + (lin & 7);
  }
  const uint32_t lds0 = lds_addr_of(lds);

  // ---- W_UV[head] -> LDS: 128 copy instructions of 1 KiB (4 rows of 256 B), 8 per wavefront.  Row c keeps its 16-byte
  // granule g at position g ^ 4*(c & 3): the transposed reads below fetch four consecutive rows per 16 lanes, and the
  // XOR spreads those rows over the banks. ----
  {
    const __bf16* w = pp.w_uv + (int64_t)head * pp.w_sn;
    const int r = lane >> 4, pos = lane & 15;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int bi = wave * 8 + i;
      const int c = 4 * bi + r;
      dma16_v(w + (int64_t)c * pp.w_sk + ((pos ^ (r << 2)) << 3), lds0 + bi * 1024);
    }
  }

  const int h32 = lane & 31, half = lane >> 5;
  for (int pass = 0; pass < pp.passes; pass++) {
    // ---- one row per wavefront: token t, this head ----
    const int t = (tb * pp.passes + pass) * kVupTok + wave;
    bool valid = t < pp.num_tokens;
    int b = 0, t_local = 0;
    if (valid) {
      int qlen;
      if (p.qsl) {
        int cnt = 0;
        for (int i = lane; i <= p.batch; i += 64) cnt += p.qsl[i] <= t ? 1 : 0;
        b = __builtin_amdgcn_readfirstlane(vup_wave_sum(cnt)) - 1;
        b = b < 0 ? 0 : (b >= p.batch ? p.batch - 1 : b);
        const int q0 = p.qsl[b];
        qlen = p.qsl[b + 1] - q0;
        t_local = t - q0;
      } else {
        b = t / p.max_q_len;
        t_local = t - b * p.max_q_len;
        qlen = p.max_q_len;
        valid = b < p.batch;
      }
      qlen = qlen < p.max_q_len ? qlen : p.max_q_len;
      valid = valid && t_local >= 0 && t_local < qlen;
    }
    float m = -INFINITY, tot = 0.f, a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (valid) vup_merge_row(p, b, t_local * p.num_heads + head, lane, m, tot, a);
    // The bf16 row goes to LDS in the order the MFMA wants its contraction index: within every 16 columns the first
    // granule holds columns {0..3, 8..11}, the second {4..7, 12..15} (the transposed reads of W deliver them in that
    // order), and granule g of row r sits at position g ^ r so that 16 rows read at the same g hit different banks.
    {
      const float inv = tot > 0.f ? 1.f / tot : 0.f;
      bf16x4 lo, hi;
#pragma unroll
      for (int e = 0; e < 4; e++) { lo[e] = (__bf16)(a[e] * inv); hi[e] = (__bf16)(a[4 + e] * inv); }
      char* rowp = lds + kVupWB + wave * 1024 + (lane & 1) * 8;
      const int g0 = (lane >> 1) * 2;
      *(bf16x4*)(rowp + (((g0) ^ wave) << 4)) = lo;
      *(bf16x4*)(rowp + (((g0 + 1) ^ wave) << 4)) = hi;
      if (lane == 0) *(int*)(lds + kVupFlagOff + wave * 4) = valid ? 1 : 0;
    }
    MLA_WAIT_VMCNT(0);                                        // this wavefront's share of W_UV has landed
    lds_barrier();

    // ---- out[t, head, 32 w .. 32 w + 31] for the pass's 16 tokens: wavefronts 0..3, 32 MFMAs each ----
    if (wave < 4) {
      const int g16 = lane >> 4, j16 = lane & 15;
      const int c_row = 4 * (g16 >> 1) + (j16 >> 2);          // row inside a group of 8 (+8 for the second read)
      const int v_cl = 2 * (g16 & 1) + ((j16 & 3) >> 1);      // granule inside this wavefront's 32 columns
      const uint32_t a_off = (uint32_t)(c_row * 256 + (((wave * 4 + v_cl) ^ ((j16 >> 2) << 2)) << 4) + (j16 & 1) * 8);
      const int tr = h32 & 15;                                // token row of the tile (lanes 16..31 repeat rows 0..15)
      const uint32_t b_off = (uint32_t)(kVupWB + tr * 1024 + ((half ^ tr) << 4));
      f32x16 acc;
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] = 0.f;
      // Operands are read with hand-placed LDS instructions kVupAhead steps ahead of the MFMA that consumes them and
      // explicit waits (three reads per step, returned in order): left to itself the compiler reads, waits and
      // multiplies one step at a time and pays the LDS latency 32 times.
      {
        const uint32_t a_lo = lds0 + a_off, a_hi = a_lo + 16 * 4096;     // the offset field holds 16 steps of 4 KiB
        const uint32_t b_ad = lds0 + b_off;
        constexpr int D = kVupAhead;
        bf16x4 wl[D], wh[D];
        bf16x8 ob[D];
#define VUP_READ(slot, kk)                                                                                             \
        do {                                                                                                           \
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(wl[slot]) : "v"((kk) < 16 ? a_lo : a_hi), "i"(((kk) & 15) * 4096)); \
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(wh[slot]) : "v"((kk) < 16 ? a_lo : a_hi), "i"(((kk) & 15) * 4096 + 2048)); \
          asm volatile("ds_read_b128 %0, %1" : "=v"(ob[slot]) : "v"(b_ad ^ (uint32_t)((kk) << 5)));                      \
        } while (0)
#pragma unroll
        for (int i = 0; i < D; i++) VUP_READ(i, i);
#pragma unroll
        for (int kk = 0; kk < 32; kk++) {
          const int younger = (31 - kk) < (D - 1) ? (31 - kk) : (D - 1);      // steps asked for after step kk
          if (younger >= 3) asm volatile("s_waitcnt lgkmcnt(9)" : "+v"(wl[kk % D]), "+v"(wh[kk % D]), "+v"(ob[kk % D]));
          else if (younger == 2) asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(wl[kk % D]), "+v"(wh[kk % D]), "+v"(ob[kk % D]));
          else if (younger == 1) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(wl[kk % D]), "+v"(wh[kk % D]), "+v"(ob[kk % D]));
          else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(wl[kk % D]), "+v"(wh[kk % D]), "+v"(ob[kk % D]));
          const bf16x8 wa = __builtin_shufflevector(wl[kk % D], wh[kk % D], 0, 1, 2, 3, 4, 5, 6, 7);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa, ob[kk % D], acc, 0, 0, 0);
          if (kk + D < 32) VUP_READ(kk % D, kk + D);
        }
#undef VUP_READ
      }
      const int tt = (tb * pp.passes + pass) * kVupTok + tr;
      const bool ok = h32 < kVupTok && *(const int*)(lds + kVupFlagOff + tr * 4) != 0;
      if (ok) {
        __bf16* o = p.out + (int64_t)tt * p.out_st + (int64_t)head * p.out_sh + wave * 32 + 4 * half;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
          bf16x4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = (__bf16)acc[q4 * 4 + e];
          *(bf16x4*)(o + q4 * 8) = v;
        }
      }
    }
    lds_barrier();                                            // the row tile is rewritten by the next pass
  }
}

int launch_reduce_vup(const ChunkReduceParams& r, const void* w_uv, int64_t w_stride_n, int64_t w_stride_k,
                      int32_t num_tokens, hipStream_t stream) {
  const int rc = ensure_dynamic_lds((const void*)mla_reduce_vup_kernel, kVupLdsB, "mla_splitkv_reduce_vup");
  if (rc != MLA_OK) return rc;
  ReduceVupParams pp;
  pp.r = r;
  pp.w_uv = (const __bf16*)w_uv; pp.w_sn = w_stride_n; pp.w_sk = w_stride_k;
  pp.num_tokens = num_tokens;
  // about one workgroup per compute unit: 16 tokens per pass, as many passes as that takes
  const int64_t blocks16 = ((int64_t)num_tokens + kVupTok - 1) / kVupTok;
  int64_t passes = (blocks16 * r.num_heads + 255) / 256;
  passes = passes < 1 ? 1 : (passes > 64 ? 64 : passes);
  pp.passes = (int32_t)passes;
  const int64_t tbs = (blocks16 + passes - 1) / passes;
  hipLaunchKernelGGL(mla_reduce_vup_kernel, dim3((unsigned)tbs, (unsigned)r.num_heads), dim3(1024), kVupLdsB, stream, pp);
  return check_launch("mla_reduce_vup_kernel");
}

}  // namespace mlahip

using namespace mlahip;

extern "C" size_t mla_decode_workspace_bytes(int32_t batch, int32_t max_q_len, int32_t num_heads, int32_t num_splits);

// Phase 2 of the split-KV decode with the value up-projection fused in: out[t, n*128 + v] for the decode tokens.
extern "C" int mla_splitkv_reduce_vup(const void* workspace, size_t workspace_bytes, const int32_t* seq_lens,
                                      const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                      int32_t num_splits, int32_t num_tokens, const void* w_uv, int64_t w_stride_n,
                                      int64_t w_stride_k, void* out, int64_t out_stride_t, int64_t out_stride_h,
                                      hipStream_t stream) {
  MLA_REQUIRE(workspace && out && seq_lens && w_uv, MLA_ERR_NULL, "mla_splitkv_reduce_vup: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_heads <= 65535 && num_splits >= 1 && num_tokens >= 0 &&
                  (int64_t)num_tokens <= (int64_t)batch * max_q_len,
              MLA_ERR_SHAPE, "mla_splitkv_reduce_vup: batch=%d max_q_len=%d num_heads=%d num_splits=%d num_tokens=%d", batch,
              max_q_len, num_heads, num_splits, num_tokens);
  MLA_REQUIRE((out_stride_t % 4 == 0) && (out_stride_h % 4 == 0) && ((uintptr_t)out % 8 == 0) &&
                  (w_stride_n % 8 == 0) && (w_stride_k % 8 == 0) && (w_stride_k >= 128) && ((uintptr_t)w_uv % 16 == 0) &&
                  ((uintptr_t)workspace % 16 == 0),
              MLA_ERR_SHAPE, "mla_splitkv_reduce_vup: W_UV rows must be 16-byte aligned, output rows 8-byte aligned");
  if (batch == 0 || num_tokens == 0) return MLA_OK;
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(workspace_bytes >= need, MLA_ERR_WORKSPACE, "mla_splitkv_reduce_vup: workspace %zu bytes < required %zu",
              workspace_bytes, need);
  const int r_max = max_q_len * num_heads;
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * r_max;
  ChunkReduceParams cp;
  cp.o_part = (const _Float16*)workspace; cp.lse_part = (const float*)((const _Float16*)workspace + rows * kDNope);
  cp.corr_scale = cp.lse_part + rows; cp.corr_row = (const __bf16* const*)(cp.lse_part + 2 * rows);
  cp.seg_ids = (const int32_t*)(cp.lse_part + 4 * rows);
  cp.seq_lens = seq_lens; cp.qsl = query_start_loc;
  cp.batch = batch; cp.max_q_len = max_q_len; cp.num_heads = num_heads; cp.num_chunks = batch * num_splits;
  cp.out = (__bf16*)out; cp.out_st = out_stride_t; cp.out_sh = out_stride_h;
  cp.lse_out = nullptr; cp.lse_st = 0;
  return launch_reduce_vup(cp, w_uv, w_stride_n, w_stride_k, num_tokens, stream);
}
