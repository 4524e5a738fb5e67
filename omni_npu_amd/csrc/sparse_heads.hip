// Sparse absorbed MLA for one query token per row list, without split-KV partials: a workgroup owns (token, 16 heads)
// and walks ALL of the token's selected keys, so the result goes straight to the output and there is nothing to merge.
//
// Replaces npu_sparse_flash_attention as the reference calls it for decode (src/omni_npu/attention/backends/dsa.py:259-291):
//   s_j = scale * (ql[t,n] . Kc[row_j] + qr[t,n] . Kr[row_j]),  o[t,n] = sum_j softmax(s)_j Kc[row_j],  j < counts[t]
// with rows[t, j] the flat cache rows that dsa_topk_rows / dsa_build_rows produced.
//
// Why this shape.  With 2048 selected keys a token is 64 blocks of 32 keys; cut into eight chunks for eight compute
// units each chunk spends more time starting and ending a segment (query staging, 128 KiB of partials) than on its
// eight blocks, and the eight partials of every row have to be merged by a second launch.  Here the eight workgroups of a
// token split the HEADS: each streams the token's 2.4 MB of selected rows through its LDS (they sit on one XCD and run in
// step, so seven of the eight find a row in that L2), keeps 16 query rows and 16 x 512 accumulators, and writes bf16.
//
// One workgroup = 8 wavefronts, tiles of 64 keys (64 x 1024 B latent + 64 x 128 B rope), two tile buffers.
//   * wavefronts 4..7 copy 16 rows of the next tile each, global -> LDS without registers, rows named by the token's row
//     list, while wavefronts 0..3 compute the scores;
//   * wavefronts 0..3 compute S^T = K Q^T for 16 keys each (18 x v_mfma_f32_16x16x32_bf16, the 16 x 576 query in 72
//     registers), P = exp2(s - reference) against a per-row reference fixed on the first tile (a score more than 2^100
//     above it makes the workgroup start over with the maxima seen so far), and publish P^T as TWO bf16 numbers per
//     probability (value and rounding remainder: 16 significant bits go through P.V);
//   * all eight wavefronts compute O^T += V^T P^T for their 64 output columns (transposed LDS reads of the same tile).
//
// Measured, 32 tokens x 128 heads x 2048 keys: 56 us, against 50 us for the split over keys + merge.  Without the copies
// the same loop takes 42 us, without the P.V MFMAs 66 (of 72 in that build), without the score MFMAs 65: the time is the
// chain barrier -> LDS reads -> dependent MFMAs -> barrier of a tile, which one wavefront per SIMD and phase does not
// hide, not matrix or memory throughput.  Two other schedules were slower: the copies shared by all eight wavefronts (0..3
// issuing theirs between their P.V MFMAs), 71 us; the tile in four column panels with wavefronts 4..7 doing P.V of
// tile t-1 and the copy of tile t+1 beside the scores of tile t, one barrier per tile, 83 us.
#include "mla_common.hpp"
#include "decode_params.hpp"

namespace mlahip {
namespace sph {

constexpr int kTile = 64;                                    // keys per tile
constexpr int kNopeB = kTile * 1024;                         // 65536
constexpr int kRopeB = kTile * 128;                          // 8192
constexpr int kBufB = kNopeB + kRopeB;                       // 73728
constexpr int kPOff = 2 * kBufB;                             // 147456: P^T, [term][k-step of 32 keys][lane][16 B] = 4 KiB
constexpr int kMaxOff = kPOff + 4096;                        // per (wave 0..3, row): row maximum of the first tile / seen maxima
constexpr int kSumOff = kMaxOff + 256;                       // per (wave 0..3, row): row sums
constexpr int kFlagOff = kSumOff + 256;                      // restart flag
constexpr int kLdsB = kFlagOff + 64;
static_assert(kLdsB <= 160 * 1024, "LDS budget");
constexpr float kRestart = 100.f;                            // log2 units above the reference

__device__ __forceinline__ int swz_nope(int r) {             // granule XOR of latent row r (16-byte granules, 64 per row)
  const int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r1 ^ r3) << 3) | (r0 << 2) | (r1 << 1) | r2;
}
__device__ __forceinline__ int swz_rope(int r) {             // granule XOR of rope row r (8 per row)
  const int r0 = r & 1, r1 = (r >> 1) & 1, r2 = (r >> 2) & 1, r3 = (r >> 3) & 1;
  return ((r0 ^ r3) << 2) | (r1 << 1) | r2;
}

struct Params {
  const __bf16* q_nope; int64_t qn_st, qn_sh;
  const __bf16* q_rope; int64_t qr_st, qr_sh;
  const __bf16* nope; int64_t nope_sr;                       // flat rows
  const __bf16* rope; int64_t rope_sr;
  int64_t max_row;
  const int32_t* rows; int64_t rows_st;
  const int32_t* counts;
  int32_t num_tokens, num_heads;
  float scale_log2;
  __bf16* out; int64_t o_st, o_sh;
  float* lse;                                                // [T, N] or null
};

__global__ __launch_bounds__(512) void dsa_sparse_heads_kernel(const Params p) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const uint32_t lds0 = lds_addr_of(lds);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
  const int l16 = lane & 15, g = lane >> 4;
  const int groups = p.num_heads >> 4;                       // head groups per token
  // the head groups of a token on one XCD (workgroups go to the eight XCDs round-robin in launch order), next to each other
  int tok, grp;
  {
    const int lin = blockIdx.x, total = p.num_tokens * groups;
    if ((p.num_tokens & 7) == 0) {
      const int xcd = lin & 7, j = lin >> 3, per = total >> 3;   // j-th workgroup of its XCD
      tok = xcd * (p.num_tokens >> 3) + j / groups;
      grp = j % groups;
      (void)per;
    } else {
      tok = lin / groups;
      grp = lin - tok * groups;
    }
  }
  int L = p.counts[tok];
  L = L < 0 ? 0 : L;
  const int tiles = (L + kTile - 1) / kTile;
  const int head0 = grp * 16;
  const bool copier = wave >= 4;
  const int cw = wave & 3;                                   // the scoring wavefront's 16 keys of a tile

  // ---- the query: 16 rows x 576 as B operands of the score MFMAs (wavefronts 0..3) ----
  // contraction step kk of the latent part covers the granules 16 * (kk % 4) + 4 g' + kk / 4 (g' = lane group): two lanes
  // 16 apart then never read one aligned 32-byte piece of a key row, which the LDS serves at half rate
  bf16x8 qf[18];
  if (!copier) {
    const __bf16* qn = p.q_nope + (int64_t)tok * p.qn_st + (int64_t)(head0 + l16) * p.qn_sh;
    const __bf16* qr = p.q_rope + (int64_t)tok * p.qr_st + (int64_t)(head0 + l16) * p.qr_sh;
#pragma unroll
    for (int kk = 0; kk < 16; kk++) qf[kk] = *(const bf16x8*)(qn + (16 * (kk & 3) + 4 * g + (kk >> 2)) * 8);
#pragma unroll
    for (int c = 0; c < 2; c++) qf[16 + c] = *(const bf16x8*)(qr + (2 * g + c) * 8);
  }

  // ---- copies (wavefronts 4..7, while 0..3 compute the scores): 16 rows of a tile each ----
  // (Shared by all eight wavefronts, with 0..3 issuing theirs between their P.V MFMAs, the step took 71 us instead of 56:
  // a copy instruction holds the issuing wavefront up for some eighty clocks, and there it sat in the phase every
  // wavefront is needed for.)
  const int32_t* my_rows = p.rows + (int64_t)tok * p.rows_st;
  auto load_ids = [&](int tile) -> int {                      // lane r < 16: cache row of key tile * 64 + 16 * cw + r
    int key = tile * kTile + cw * 16 + l16;
    key = key < L ? key : L - 1;
    key = key < 0 ? 0 : key;
    int64_t r = my_rows[key];
    r = r < 0 ? 0 : (r > p.max_row ? p.max_row : r);
    return (int)r;
  };
  const uint32_t n_sr2 = (uint32_t)p.nope_sr * 2u, r_sr2 = (uint32_t)p.rope_sr * 2u;
  auto issue_tile = [&](int tile, int ids) {
    const uint32_t buf = lds0 + (tile & 1) * kBufB;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int64_t id = __builtin_amdgcn_readlane(ids, i);
      dma16_sv((const char*)p.nope + id * n_sr2, (uint32_t)((lane ^ swz_nope(i)) << 4), buf + (cw * 16 + i) * 1024);
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const int rl = 8 * j + (lane >> 3);                     // this lane's row among the wave's 16
      const int64_t id = __shfl(ids, rl, 64);
      dma16_v((const char*)p.rope + id * r_sr2 + (((lane & 7) ^ swz_rope(rl)) << 4), buf + kNopeB + (cw * 16 + 8 * j) * 128);
    }
  };

  // ---- per-lane LDS offsets ----
  // scores: lane (key l16 of the wave's 16, group g) reads 16 bytes of key row 16 * wave + l16
  int koff[4];                                               // latent granules 4g + c of quarter 16 * (kk % 4): c = kk / 4
#pragma unroll
  for (int c = 0; c < 4; c++) koff[c] = (cw * 16 + l16) * 1024 + (((4 * g + c) ^ swz_nope(l16)) << 4);   // ^ (16 * (kk % 4)) << 4
  int roff[2];
#pragma unroll
  for (int c = 0; c < 2; c++) roff[c] = kNopeB + (cw * 16 + l16) * 128 + (((2 * g + c) ^ swz_rope(l16)) << 4);
  // P.V: V^T fragment of (k-step ks, column tile dt) = two transposed reads; lane (g, j = l16) points at key
  // 32 ks + 4 g + (j >> 2) (+ 16) and the 8 bytes (j & 3) of the 32 bytes of columns [64 wave + 16 dt, + 16)
  int voff[2];                                               // [lower / upper 16 keys of the k-step], + ks * 32 * 1024, ^ granule of dt
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int rr = 16 * h + 4 * g + (l16 >> 2);              // key row inside the k-step (the swizzle sees rr % 16)
    voff[h] = rr * 1024 + (l16 & 1) * 8 + (((8 * wave + ((l16 & 3) >> 1)) ^ swz_nope(rr & 15)) << 4);
  }

  f32x4 acc[4];
  float m_ref = -INFINITY, l_run = 0.f, m_seen = -INFINITY;
  int ids_cur = 0;
  auto prime = [&] {                                          // (copying wavefronts) tile 0 on its way, the rows of tile 1 at hand
    if (copier && tiles > 0) {
      ids_cur = load_ids(0);
      issue_tile(0, ids_cur);
      if (tiles > 1) ids_cur = load_ids(1);
    }
  };
  prime();
  if (threadIdx.x == 0) *(int*)(lds + kFlagOff) = 0;

  for (int attempt = 0; attempt < 2 && tiles > 0; attempt++) {
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    l_run = 0.f;
    for (int tile = 0; tile < tiles; tile++) {
      const char* buf = lds + (tile & 1) * kBufB;
      // tile `tile` has landed, everyone is done with the other buffer and with the P of the previous tile
      MLA_WAIT_VMCNT(0);
      lds_barrier();
      float sc[4] = {0.f, 0.f, 0.f, 0.f};
      if (copier) {
        if (tile + 1 < tiles) {
          const int ids_next = tile + 2 < tiles ? load_ids(tile + 2) : 0;
          issue_tile(tile + 1, ids_cur);
          ids_cur = ids_next;
        }
      } else {
        // ---- scores of this wave's 16 keys x 16 rows (three accumulators: a chain of 18 dependent MFMAs would wait for
        // each one's result) ----
        f32x4 s3[3];
#pragma unroll
        for (int i = 0; i < 3; i++) s3[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
          const bf16x8 a = *(const bf16x8*)(buf + (koff[kk >> 2] ^ ((16 * (kk & 3)) << 4)));
          s3[kk % 3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[kk], s3[kk % 3], 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < 2; c++) {
          const bf16x8 a = *(const bf16x8*)(buf + roff[c]);
          s3[(16 + c) % 3] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[16 + c], s3[(16 + c) % 3], 0, 0, 0);
        }
        const f32x4 s = (s3[0] + s3[1]) + s3[2];
        // lane (row l16, group g) holds keys tile * 64 + 16 * wave + 4 g + r; keys past the list's end weigh nothing
        const int key0 = tile * kTile + 16 * cw + 4 * g;
#pragma unroll
        for (int r = 0; r < 4; r++) sc[r] = key0 + r < L ? s[r] * p.scale_log2 : -INFINITY;
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));               // the row's maximum over this wave's 16 keys
        m_seen = fmaxf(m_seen, mx);
        if (attempt == 0 && tile == 0 && g == 0) *(float*)(lds + kMaxOff + (cw * 16 + l16) * 4) = mx;
      }
      if (attempt == 0 && tile == 0) {
        // the first tile fixes every row's reference: its maximum over the tile's 64 keys (the four scoring wavefronts)
        lds_barrier();
        if (!copier) {
          const float* mm = (const float*)(lds + kMaxOff);
          m_ref = fmaxf(fmaxf(mm[l16], mm[16 + l16]), fmaxf(mm[32 + l16], mm[48 + l16]));
        }
      }
      if (!copier) {
        float pr[4];
        bool high = false;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float t = sc[r] - m_ref;
          high |= t > kRestart;
          pr[r] = fast_exp2(t);                               // exp2(-inf) = 0 for the masked keys
          l_run += pr[r];
        }
        if (__builtin_amdgcn_ballot_w64(high) != 0 && lane == 0) *(volatile int*)(lds + kFlagOff) = 1;
        // P^T as two bf16 numbers per probability, where the P.V operand of k-step cw / 2 wants them: lane (row, g) there
        // holds keys {4 g + r} of the step's lower 16 keys and of its upper 16 keys, i.e. this wave's and its neighbour's
        bf16x4 hi, lo;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          hi[r] = (__bf16)pr[r];
          lo[r] = (__bf16)(pr[r] - (float)hi[r]);
        }
        char* pp = lds + kPOff + (cw >> 1) * 1024 + lane * 16 + (cw & 1) * 8;
        *(bf16x4*)pp = hi;
        *(bf16x4*)(pp + 2048) = lo;
      }
      lds_barrier();
      // ---- O^T += V^T P^T: this wave's 64 columns, all 16 rows ----
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        const bf16x8 p_hi = *(const bf16x8*)(lds + kPOff + ks * 1024 + lane * 16);
        const bf16x8 p_lo = *(const bf16x8*)(lds + kPOff + 2048 + ks * 1024 + lane * 16);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          const bf16x4 v0 = lds_read_tr16(buf + ks * 32 * 1024 + (voff[0] ^ ((2 * dt) << 4)));
          const bf16x4 v1 = lds_read_tr16(buf + ks * 32 * 1024 + (voff[1] ^ ((2 * dt) << 4)));
          const bf16x8 a = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p_hi, acc[dt], 0, 0, 0);
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p_lo, acc[dt], 0, 0, 0);
        }
      }
    }
    // a score that outgrew its reference by more than 2^100: once more, with the maxima of the whole pass as references
    // (they are the true maxima, so the second pass cannot ask again)
    lds_barrier();
    const int flag = *(volatile int*)(lds + kFlagOff);
    if (flag == 0) break;
    if (!copier && g == 0) *(float*)(lds + kMaxOff + (cw * 16 + l16) * 4) = m_seen;
    lds_barrier();
    if (threadIdx.x == 0) *(volatile int*)(lds + kFlagOff) = 0;
    if (!copier) {
      const float* mm = (const float*)(lds + kMaxOff);
      m_ref = fmaxf(fmaxf(mm[l16], mm[16 + l16]), fmaxf(mm[32 + l16], mm[48 + l16]));
    }
    prime();
  }

  // ---- the rows' sums, then the normalised result ----
  if (!copier) {
    float lt = l_run + __shfl_xor(l_run, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (g == 0) *(float*)(lds + kSumOff + (cw * 16 + l16) * 4) = lt;
  }
  lds_barrier();
  const float* ss = (const float*)(lds + kSumOff);
  const float l_tot = tiles > 0 ? (ss[l16] + ss[16 + l16]) + (ss[32 + l16] + ss[48 + l16]) : 0.f;
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  __bf16* o = p.out + (int64_t)tok * p.o_st + (int64_t)(head0 + l16) * p.o_sh + 64 * wave + 4 * g;
#pragma unroll
  for (int dt = 0; dt < 4; dt++) {
    bf16x4 v;
#pragma unroll
    for (int r = 0; r < 4; r++) v[r] = (__bf16)(tiles > 0 ? acc[dt][r] * inv : 0.f);
    *(bf16x4*)(o + 16 * dt) = v;
  }
  if (p.lse && wave == 0 && g == 0)
    p.lse[(int64_t)tok * p.num_heads + head0 + l16] = l_tot > 0.f ? (m_ref + fast_log2(l_tot)) * kLn2 : -INFINITY;
}

}  // namespace sph
}  // namespace mlahip
using namespace mlahip;

// Sparse absorbed MLA, one launch, no workspace: token t attends to the cache rows sparse_rows[t, 0 .. counts[t]) (flat row
// numbers, pages contiguous) - the arithmetic of dsa_sparse_decode_bf16 with the work split over heads instead of keys.
// num_heads must be a multiple of 16; out bf16 [T,N,512] through its strides, lse_out fp32 [T,N] or NULL.
extern "C" int dsa_sparse_decode_heads_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                            int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                            int64_t nope_row_stride, const void* rope_cache, int64_t rope_row_stride,
                                            int64_t num_rows, const int32_t* sparse_rows, int64_t sparse_stride,
                                            const int32_t* counts, int32_t num_tokens, int32_t num_heads, float scale,
                                            void* out, int64_t out_stride_t, int64_t out_stride_h, float* lse_out,
                                            hipStream_t stream) {
  MLA_REQUIRE(q_nope && q_rope && nope_cache && rope_cache && sparse_rows && counts && out, MLA_ERR_NULL,
              "dsa_sparse_decode_heads_bf16: null pointer argument");
  MLA_REQUIRE(num_tokens >= 0 && num_heads >= 16 && num_heads % 16 == 0 && num_rows >= 1 && sparse_stride >= 1, MLA_ERR_SHAPE,
              "dsa_sparse_decode_heads_bf16: num_tokens=%d num_heads=%d (a multiple of 16) num_rows=%lld", num_tokens, num_heads,
              (long long)num_rows);
  MLA_REQUIRE((int64_t)num_tokens * (num_heads / 16) <= 0x7fffffff, MLA_ERR_SHAPE, "dsa_sparse_decode_heads_bf16: grid limit exceeded");
  MLA_REQUIRE(qn_stride_t % 8 == 0 && qn_stride_h % 8 == 0 && qr_stride_t % 8 == 0 && qr_stride_h % 8 == 0 &&
                  nope_row_stride % 8 == 0 && rope_row_stride % 8 == 0 && out_stride_t % 4 == 0 && out_stride_h % 4 == 0 &&
                  nope_row_stride < (1 << 28) && rope_row_stride < (1 << 28),
              MLA_ERR_SHAPE, "dsa_sparse_decode_heads_bf16: strides must keep 16-byte alignment of 8-element groups");
  MLA_REQUIRE((uintptr_t)q_nope % 16 == 0 && (uintptr_t)q_rope % 16 == 0 && (uintptr_t)nope_cache % 16 == 0 &&
                  (uintptr_t)rope_cache % 16 == 0 && (uintptr_t)out % 8 == 0,
              MLA_ERR_SHAPE, "dsa_sparse_decode_heads_bf16: pointers must be 16-byte aligned");
  MLA_REQUIRE(scale > 0.f, MLA_ERR_UNSUPPORTED, "dsa_sparse_decode_heads_bf16: the softmax scale must be positive");
  if (num_tokens == 0) return MLA_OK;
  sph::Params p;
  p.q_nope = (const __bf16*)q_nope; p.qn_st = qn_stride_t; p.qn_sh = qn_stride_h;
  p.q_rope = (const __bf16*)q_rope; p.qr_st = qr_stride_t; p.qr_sh = qr_stride_h;
  p.nope = (const __bf16*)nope_cache; p.nope_sr = nope_row_stride;
  p.rope = (const __bf16*)rope_cache; p.rope_sr = rope_row_stride;
  p.max_row = num_rows - 1;
  p.rows = sparse_rows; p.rows_st = sparse_stride; p.counts = counts;
  p.num_tokens = num_tokens; p.num_heads = num_heads;
  p.scale_log2 = scale * kLog2e;
  p.out = (__bf16*)out; p.o_st = out_stride_t; p.o_sh = out_stride_h; p.lse = lse_out;
  const int rc = ensure_dynamic_lds((const void*)sph::dsa_sparse_heads_kernel, sph::kLdsB, "dsa_sparse_heads_kernel");
  if (rc != MLA_OK) return rc;
  hipLaunchKernelGGL(sph::dsa_sparse_heads_kernel, dim3((unsigned)(num_tokens * (num_heads / 16))), dim3(512), sph::kLdsB, stream, p);
  return check_launch("dsa_sparse_heads_kernel");
}
