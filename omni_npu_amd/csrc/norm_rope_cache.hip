// The step in front of the attention kernels, fused: RMSNorm of the compressed KV (512), rotary embedding of the shared
// rope key (64) and the write of both into the paged cache; plus the rotary embedding of the query's rope part.
//
// Replaces torch_npu.npu_kv_rmsnorm_rope_cache as called at
//   src/omni_npu/v1/layers/attention/npu_mla.py:196-206, 296-309 and src/omni_npu/v1/layers/attention/npu_dsa.py:410-424,
//   517-527 (kv [T,1,1,576], gamma [512], cos / sin [T,1,1,64], slot_mapping [T], the two caches; optional k_pe / kv_a
//   outputs when is_output_kv is set)
// and torch_npu.npu_interleave_rope (npu_mla.py:210, 316; npu_dsa.py:407, 528).  The arithmetic is the reference's own
// torch formulation of the same ops:
//   RMSNorm   y = x * rsqrt(mean(x^2) + eps) * gamma                       (the kv_a_layernorm of npu_dsa.py:405)
//   rotary    x1 = x[0::2], x2 = x[1::2];  o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin;  out = cat(o1, o2)
//             (src/omni_npu/layers/rotary_embedding/rotary_embedding_torch_npu.py:146-163, the non-neox branch that the
//             vendor op stands in for; cos / sin rows there are cat(c, c), 64 wide: pair i uses entry i)
// computed in fp32 from the bf16 inputs and rounded to bf16 once.  The output of the rotation is DE-INTERLEAVED (all
// o1 first), as in the reference; `interleaved_out` keeps the pairs in place instead (the GPT-J convention of
// tests/integration/attention/test_npu_mla_math.py:125-144, whose tables repeat every entry: cos_step = 2).
//
// One wavefront per token: lane l owns latent elements [8l, 8l+8), lanes 0..7 own four rope pairs each.  The fp8 variant
// quantises the bf16-rounded normalised row exactly as mla_cache_write_fp8 does (656-byte rows).
#include "mla_common.hpp"

// every product and sum below is rounded on its own: results must not depend on what the compiler chooses to fuse
#pragma clang fp contract(off)

namespace mlahip {

constexpr int kF8RowB = 656, kF8ScaleOff = 512, kF8RopeOff = 528;

struct NormRopeParams {
  const __bf16* kv_a; int64_t kv_a_stride;        // [T, 512]
  const __bf16* k_pe; int64_t k_pe_stride;        // [T, 64]
  const __bf16* gamma;                            // [512]
  const __bf16* cos; const __bf16* sin; int64_t cs_stride; int32_t cos_step;
  const int64_t* slots; int32_t num_tokens;
  float eps;
  int32_t interleaved_out;
  char* nope_cache; int64_t nope_sp, nope_sr;     // bytes; in fp8 mode the one 656-byte-row cache
  char* rope_cache; int64_t rope_sp, rope_sr;
  int32_t page_size; int64_t num_pages;
  __bf16* kv_a_out; int64_t kv_a_out_stride;      // optional [T, 512]
  __bf16* k_pe_out; int64_t k_pe_out_stride;      // optional [T, 64]
};

// Rotates four pairs: x holds elements [8j, 8j+8) of a 64-wide rope vector, c / s point at the token's table rows.
// Returns o1 (pairs' first results) and o2 as packed bf16.
__device__ __forceinline__ void rope4(const bf16x8& x, const __bf16* c, const __bf16* s, int pair0, int step, bf16x4& o1,
                                      bf16x4& o2) {
#pragma unroll
  for (int e = 0; e < 4; e++) {
    const float cc = (float)c[(pair0 + e) * step], ss = (float)s[(pair0 + e) * step];
    const float x1 = (float)x[2 * e], x2 = (float)x[2 * e + 1];
    // products rounded separately (no contraction), so that the result does not depend on how the compiler fuses them
    const float a = __fmul_rn(x1, cc), b = __fmul_rn(x2, ss), d = __fmul_rn(x2, cc), g = __fmul_rn(x1, ss);
    o1[e] = (__bf16)__fsub_rn(a, b);
    o2[e] = (__bf16)__fadd_rn(d, g);
  }
}

template <bool kFp8>
__device__ __forceinline__ void kv_norm_rope_body(const NormRopeParams& p, int64_t block) {
  const int lane = threadIdx.x & 63;
  const int64_t t = block * 4 + (threadIdx.x >> 6);
  if (t >= p.num_tokens) return;
  const int64_t slot = p.slots ? p.slots[t] : -1;
  const bool store = slot >= 0 && slot < p.num_pages * p.page_size;
  if (!store && !p.kv_a_out && !p.k_pe_out) return;
  const int64_t pg = store ? slot / p.page_size : 0;
  const int64_t off = store ? slot - pg * p.page_size : 0;

  // ---- RMSNorm of the latent part ----
  const bf16x8 v = *(const bf16x8*)(p.kv_a + t * p.kv_a_stride + lane * 8);
  const bf16x8 g = *(const bf16x8*)(p.gamma + lane * 8);
  float x[8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) { x[e] = (float)v[e]; ss = __fadd_rn(ss, __fmul_rn(x[e], x[e])); }
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) ss = __fadd_rn(ss, __shfl_xor(ss, o, 64));   // same total in every lane, fixed order
  const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(__fmul_rn(ss, 1.0f / 512.0f), p.eps)));
  bf16x8 y;
#pragma unroll
  for (int e = 0; e < 8; e++) y[e] = (__bf16)__fmul_rn(__fmul_rn(x[e], inv), (float)g[e]);
  if (p.kv_a_out) *(bf16x8*)(p.kv_a_out + t * p.kv_a_out_stride + lane * 8) = y;

  if (store) {
    if constexpr (kFp8) {
      char* row = p.nope_cache + pg * p.nope_sp + off * p.nope_sr;
      float f[8];
      float amax = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) { f[e] = (float)y[e]; amax = fmaxf(amax, fabsf(f[e])); }
#pragma unroll
      for (int o = 1; o < 16; o <<= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));   // 16 lanes = one 128-element block
      const float scale = amax > 0.f ? amax / 448.f : 1.f;
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] = fminf(fmaxf(f[e] / scale, -448.f), 448.f);
      int w0 = 0, w1 = 0;
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], w0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], w0, true);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], w1, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], w1, true);
      const u32x2 packed = {(uint32_t)w0, (uint32_t)w1};
      *(u32x2*)(row + lane * 8) = packed;
      if ((lane & 15) == 0) *(float*)(row + kF8ScaleOff + (lane >> 4) * 4) = scale;
    } else {
      *(bf16x8*)(p.nope_cache + pg * p.nope_sp + off * p.nope_sr + lane * 16) = y;
    }
  }

  // ---- rotary embedding of the rope part: lanes 0..7, four pairs each ----
  if (lane < 8) {
    const bf16x8 r = *(const bf16x8*)(p.k_pe + t * p.k_pe_stride + lane * 8);
    bf16x4 o1, o2;
    rope4(r, p.cos + t * p.cs_stride, p.sin + t * p.cs_stride, lane * 4, p.cos_step, o1, o2);
    char* dst = nullptr;
    if (store) dst = kFp8 ? p.nope_cache + pg * p.nope_sp + off * p.nope_sr + kF8RopeOff
                          : p.rope_cache + pg * p.rope_sp + off * p.rope_sr;
    char* dst2 = p.k_pe_out ? (char*)(p.k_pe_out + t * p.k_pe_out_stride) : nullptr;
    if (p.interleaved_out) {
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 4; e++) { o[2 * e] = o1[e]; o[2 * e + 1] = o2[e]; }
      if (dst) *(bf16x8*)(dst + lane * 16) = o;
      if (dst2) *(bf16x8*)(dst2 + lane * 16) = o;
    } else {
      if (dst) { *(bf16x4*)(dst + lane * 8) = o1; *(bf16x4*)(dst + 64 + lane * 8) = o2; }
      if (dst2) { *(bf16x4*)(dst2 + lane * 8) = o1; *(bf16x4*)(dst2 + 64 + lane * 8) = o2; }
    }
  }
}

template <bool kFp8>
__global__ __launch_bounds__(256) void kv_rmsnorm_rope_cache_kernel(NormRopeParams p) {
  kv_norm_rope_body<kFp8>(p, blockIdx.x);
}

struct RopeParams {
  const __bf16* x; int64_t x_st, x_sh;
  __bf16* out; int64_t o_st, o_sh;
  const __bf16* cos; const __bf16* sin; int64_t cs_stride; int32_t cos_step;
  int64_t num_tokens; int32_t num_heads; int32_t interleaved_out;
};

// One thread per (token, head, group of four pairs).
__device__ __forceinline__ void interleave_rope_body(const RopeParams& p, int64_t block) {
  const int64_t i = block * 256 + threadIdx.x;
  const int j = (int)(i & 7);
  const int64_t th = i >> 3;
  const int64_t t = th / p.num_heads;
  const int h = (int)(th - t * p.num_heads);
  if (t >= p.num_tokens) return;
  const bf16x8 r = *(const bf16x8*)(p.x + t * p.x_st + (int64_t)h * p.x_sh + j * 8);
  bf16x4 o1, o2;
  rope4(r, p.cos + t * p.cs_stride, p.sin + t * p.cs_stride, j * 4, p.cos_step, o1, o2);
  char* dst = (char*)(p.out + t * p.o_st + (int64_t)h * p.o_sh);
  if (p.interleaved_out) {
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 4; e++) { o[2 * e] = o1[e]; o[2 * e + 1] = o2[e]; }
    *(bf16x8*)(dst + j * 16) = o;
  } else {
    *(bf16x4*)(dst + j * 8) = o1;
    *(bf16x4*)(dst + 64 + j * 8) = o2;
  }
}

__global__ __launch_bounds__(256) void interleave_rope_kernel(RopeParams p) { interleave_rope_body(p, blockIdx.x); }

// Both in one launch (the decode step's prologue: a handful of tokens, launch latency is all there is): the first
// kv_blocks workgroups normalise, rotate and store the keys, the others rotate the query's rope part.
template <bool kFp8>
__global__ __launch_bounds__(256) void kv_q_prologue_kernel(NormRopeParams p, RopeParams q, int32_t kv_blocks) {
  if ((int)blockIdx.x < kv_blocks) kv_norm_rope_body<kFp8>(p, blockIdx.x);
  else interleave_rope_body(q, (int64_t)blockIdx.x - kv_blocks);
}

// Half-rotation ("neox") pairing: element i pairs with element i + 32, the result keeps the input's layout, so the
// rotation may run in place.  One thread per (token, head, group of four pairs).
__global__ __launch_bounds__(256) void rotary_mul_kernel(RopeParams p) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int j = (int)(i & 7);
  const int64_t th = i >> 3;
  const int64_t t = th / p.num_heads;
  const int h = (int)(th - t * p.num_heads);
  if (t >= p.num_tokens) return;
  const __bf16* src = p.x + t * p.x_st + (int64_t)h * p.x_sh;
  const bf16x4 a = *(const bf16x4*)(src + j * 4), b = *(const bf16x4*)(src + 32 + j * 4);
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 4; e++) { r[2 * e] = a[e]; r[2 * e + 1] = b[e]; }
  bf16x4 o1, o2;
  rope4(r, p.cos + t * p.cs_stride, p.sin + t * p.cs_stride, j * 4, p.cos_step, o1, o2);
  char* dst = (char*)(p.out + t * p.o_st + (int64_t)h * p.o_sh);
  *(bf16x4*)(dst + j * 8) = o1;
  *(bf16x4*)(dst + 64 + j * 8) = o2;
}

static int check_tables(const char* who, const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step) {
  MLA_REQUIRE(cos && sin, MLA_ERR_NULL, "%s: null cos / sin table", who);
  MLA_REQUIRE((cos_step == 1 || cos_step == 2) && cs_stride >= 31 * (int64_t)cos_step + 1, MLA_ERR_SHAPE,
              "%s: cos_step must be 1 or 2 and a table row must hold 32 entries at that step (stride %lld)", who,
              (long long)cs_stride);
  return MLA_OK;
}

static int norm_rope_impl(bool fp8, const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                          const void* gamma, const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step,
                          int32_t interleaved_out, const int64_t* slot_mapping, int32_t num_tokens, float eps,
                          void* nope_cache, int64_t nope_sp_b, int64_t nope_sr_b, void* rope_cache, int64_t rope_sp_b,
                          int64_t rope_sr_b, int32_t page_size, int64_t num_pages, void* kv_a_out,
                          int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride, hipStream_t stream,
                          const RopeParams* q = nullptr) {
  const char* who = fp8 ? (q ? "mla_kv_rmsnorm_rope_cache_q_fp8" : "mla_kv_rmsnorm_rope_cache_fp8")
                        : (q ? "mla_kv_rmsnorm_rope_cache_q" : "mla_kv_rmsnorm_rope_cache");
  // without a slot mapping nothing is cached: the normalised latent and the rotated key only go to the plain outputs
  MLA_REQUIRE(kv_a && k_pe && gamma && (slot_mapping ? (nope_cache && (fp8 || rope_cache)) : (kv_a_out && k_pe_out)),
              MLA_ERR_NULL, "%s: null pointer argument", who);
  if (int rc = check_tables(who, cos, sin, cs_stride, cos_step)) return rc;
  MLA_REQUIRE(num_tokens >= 0 && (!slot_mapping || (page_size >= 1 && num_pages >= 1)) && eps >= 0.f, MLA_ERR_SHAPE,
              "%s: num_tokens=%d page_size=%d num_pages=%lld eps=%g", who, num_tokens, page_size, (long long)num_pages,
              (double)eps);
  MLA_REQUIRE(kv_a_stride % 8 == 0 && k_pe_stride % 8 == 0 && (uintptr_t)kv_a % 16 == 0 && (uintptr_t)k_pe % 16 == 0 &&
                  (uintptr_t)gamma % 16 == 0 &&
                  (!slot_mapping || (nope_sp_b % 16 == 0 && nope_sr_b % 16 == 0 && (uintptr_t)nope_cache % 16 == 0 &&
                                     (fp8 || (rope_sp_b % 16 == 0 && rope_sr_b % 16 == 0 && (uintptr_t)rope_cache % 16 == 0)))) &&
                  (!kv_a_out || (kv_a_out_stride % 8 == 0 && (uintptr_t)kv_a_out % 16 == 0)) &&
                  (!k_pe_out || (k_pe_out_stride % 8 == 0 && (uintptr_t)k_pe_out % 16 == 0)),
              MLA_ERR_SHAPE, "%s: rows must be 16-byte aligned", who);
  MLA_REQUIRE(!fp8 || !slot_mapping || nope_sr_b >= kF8RowB, MLA_ERR_SHAPE, "%s: fp8 cache rows are 656 bytes", who);
  if (num_tokens == 0) return MLA_OK;
  NormRopeParams p;
  p.kv_a = (const __bf16*)kv_a; p.kv_a_stride = kv_a_stride; p.k_pe = (const __bf16*)k_pe; p.k_pe_stride = k_pe_stride;
  p.gamma = (const __bf16*)gamma; p.cos = (const __bf16*)cos; p.sin = (const __bf16*)sin; p.cs_stride = cs_stride;
  p.cos_step = cos_step; p.slots = slot_mapping; p.num_tokens = num_tokens; p.eps = eps; p.interleaved_out = interleaved_out;
  p.nope_cache = (char*)nope_cache; p.nope_sp = nope_sp_b; p.nope_sr = nope_sr_b;
  p.rope_cache = (char*)rope_cache; p.rope_sp = rope_sp_b; p.rope_sr = rope_sr_b;
  p.page_size = page_size; p.num_pages = num_pages;
  p.kv_a_out = (__bf16*)kv_a_out; p.kv_a_out_stride = kv_a_out_stride;
  p.k_pe_out = (__bf16*)k_pe_out; p.k_pe_out_stride = k_pe_out_stride;
  const dim3 grid((unsigned)((num_tokens + 3) / 4));
  if (q) {
    const int64_t q_blocks = (q->num_tokens * q->num_heads * 8 + 255) / 256;
    MLA_REQUIRE((int64_t)grid.x + q_blocks < (1ll << 31), MLA_ERR_SHAPE, "%s: too many rows for one launch", who);
    const dim3 both((unsigned)(grid.x + q_blocks));
    if (fp8) hipLaunchKernelGGL(kv_q_prologue_kernel<true>, both, dim3(256), 0, stream, p, *q, (int32_t)grid.x);
    else hipLaunchKernelGGL(kv_q_prologue_kernel<false>, both, dim3(256), 0, stream, p, *q, (int32_t)grid.x);
    return check_launch(who);
  }
  if (fp8) hipLaunchKernelGGL(kv_rmsnorm_rope_cache_kernel<true>, grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(kv_rmsnorm_rope_cache_kernel<false>, grid, dim3(256), 0, stream, p);
  return check_launch(who);
}

// Argument checks and parameters of the query rotation shared by mla_interleave_rope and the fused prologue entries.
static int rope_params(const char* who, const void* x, int64_t x_stride_t, int64_t x_stride_h, int64_t num_tokens,
                       int32_t num_heads, const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step,
                       int32_t interleaved_out, void* out, int64_t out_stride_t, int64_t out_stride_h, RopeParams* p) {
  MLA_REQUIRE(x && out, MLA_ERR_NULL, "%s: null pointer argument", who);
  if (int rc = check_tables(who, cos, sin, cs_stride, cos_step)) return rc;
  MLA_REQUIRE(num_tokens >= 0 && num_heads >= 1 && num_tokens * num_heads < (1ll << 40), MLA_ERR_SHAPE,
              "%s: num_tokens=%lld num_heads=%d", who, (long long)num_tokens, num_heads);
  MLA_REQUIRE(x_stride_t % 8 == 0 && x_stride_h % 8 == 0 && out_stride_t % 8 == 0 && out_stride_h % 8 == 0 &&
                  (uintptr_t)x % 16 == 0 && (uintptr_t)out % 16 == 0,
              MLA_ERR_SHAPE, "%s: query rows must be 16-byte aligned", who);
  // In place (out == x, same strides) is fine in both output layouts: the eight threads of a row are neighbouring lanes
  // of one wavefront, whose load instruction has returned for all of them before its store instruction is issued.
  MLA_REQUIRE(x != out || (x_stride_t == out_stride_t && x_stride_h == out_stride_h), MLA_ERR_UNSUPPORTED,
              "%s: in place needs the same strides for x and out", who);
  p->x = (const __bf16*)x; p->x_st = x_stride_t; p->x_sh = x_stride_h; p->out = (__bf16*)out; p->o_st = out_stride_t;
  p->o_sh = out_stride_h; p->cos = (const __bf16*)cos; p->sin = (const __bf16*)sin; p->cs_stride = cs_stride;
  p->cos_step = cos_step; p->num_tokens = num_tokens; p->num_heads = num_heads; p->interleaved_out = interleaved_out;
  return MLA_OK;
}

}  // namespace mlahip
using namespace mlahip;

extern "C" int mla_kv_rmsnorm_rope_cache(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                         const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                         int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                         int32_t num_tokens, float eps, void* nope_cache, int64_t nope_page_stride,
                                         int64_t nope_row_stride, void* rope_cache, int64_t rope_page_stride,
                                         int64_t rope_row_stride, int32_t page_size, int64_t num_pages, void* kv_a_out,
                                         int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride,
                                         hipStream_t stream) {
  MLA_REQUIRE(nope_page_stride % 8 == 0 && nope_row_stride % 8 == 0 && rope_page_stride % 8 == 0 && rope_row_stride % 8 == 0,
              MLA_ERR_SHAPE, "mla_kv_rmsnorm_rope_cache: cache strides must be multiples of 8 elements");
  return norm_rope_impl(false, kv_a, kv_a_stride, k_pe, k_pe_stride, gamma, cos, sin, cs_stride, cos_step, interleaved_out,
                        slot_mapping, num_tokens, eps, nope_cache, nope_page_stride * 2, nope_row_stride * 2, rope_cache,
                        rope_page_stride * 2, rope_row_stride * 2, page_size, num_pages, kv_a_out, kv_a_out_stride, k_pe_out,
                        k_pe_out_stride, stream);
}

extern "C" int mla_kv_rmsnorm_rope_cache_fp8(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                             const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                             int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                             int32_t num_tokens, float eps, void* cache, int64_t page_stride_bytes,
                                             int64_t row_stride_bytes, int32_t page_size, int64_t num_pages,
                                             void* kv_a_out, int64_t kv_a_out_stride, void* k_pe_out,
                                             int64_t k_pe_out_stride, hipStream_t stream) {
  return norm_rope_impl(true, kv_a, kv_a_stride, k_pe, k_pe_stride, gamma, cos, sin, cs_stride, cos_step, interleaved_out,
                        slot_mapping, num_tokens, eps, cache, page_stride_bytes, row_stride_bytes, nullptr, 0, 0, page_size,
                        num_pages, kv_a_out, kv_a_out_stride, k_pe_out, k_pe_out_stride, stream);
}

extern "C" int mla_interleave_rope(const void* x, int64_t x_stride_t, int64_t x_stride_h, int64_t num_tokens,
                                   int32_t num_heads, const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step,
                                   int32_t interleaved_out, void* out, int64_t out_stride_t, int64_t out_stride_h,
                                   hipStream_t stream) {
  RopeParams p;
  if (int rc = rope_params("mla_interleave_rope", x, x_stride_t, x_stride_h, num_tokens, num_heads, cos, sin, cs_stride,
                           cos_step, interleaved_out, out, out_stride_t, out_stride_h, &p))
    return rc;
  if (num_tokens == 0) return MLA_OK;
  const int64_t threads = num_tokens * num_heads * 8;
  hipLaunchKernelGGL(interleave_rope_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, p);
  return check_launch("mla_interleave_rope");
}

// mla_kv_rmsnorm_rope_cache and mla_interleave_rope of the same tokens (same tables, same output convention) in one launch.
extern "C" int mla_kv_rmsnorm_rope_cache_q(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                           const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                           int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                           int32_t num_tokens, float eps, void* nope_cache, int64_t nope_page_stride,
                                           int64_t nope_row_stride, void* rope_cache, int64_t rope_page_stride,
                                           int64_t rope_row_stride, int32_t page_size, int64_t num_pages, void* kv_a_out,
                                           int64_t kv_a_out_stride, void* k_pe_out, int64_t k_pe_out_stride, const void* q,
                                           int64_t q_stride_t, int64_t q_stride_h, int32_t num_heads, void* q_out,
                                           int64_t q_out_stride_t, int64_t q_out_stride_h, hipStream_t stream) {
  MLA_REQUIRE(nope_page_stride % 8 == 0 && nope_row_stride % 8 == 0 && rope_page_stride % 8 == 0 && rope_row_stride % 8 == 0,
              MLA_ERR_SHAPE, "mla_kv_rmsnorm_rope_cache_q: cache rows must be 16-byte aligned");
  RopeParams qp;
  if (int rc = rope_params("mla_kv_rmsnorm_rope_cache_q", q, q_stride_t, q_stride_h, num_tokens, num_heads, cos, sin, cs_stride,
                           cos_step, interleaved_out, q_out, q_out_stride_t, q_out_stride_h, &qp))
    return rc;
  return norm_rope_impl(false, kv_a, kv_a_stride, k_pe, k_pe_stride, gamma, cos, sin, cs_stride, cos_step, interleaved_out,
                        slot_mapping, num_tokens, eps, nope_cache, nope_page_stride * 2, nope_row_stride * 2, rope_cache,
                        rope_page_stride * 2, rope_row_stride * 2, page_size, num_pages, kv_a_out, kv_a_out_stride, k_pe_out,
                        k_pe_out_stride, stream, &qp);
}

extern "C" int mla_kv_rmsnorm_rope_cache_q_fp8(const void* kv_a, int64_t kv_a_stride, const void* k_pe, int64_t k_pe_stride,
                                               const void* gamma, const void* cos, const void* sin, int64_t cs_stride,
                                               int32_t cos_step, int32_t interleaved_out, const int64_t* slot_mapping,
                                               int32_t num_tokens, float eps, void* cache, int64_t page_stride_bytes,
                                               int64_t row_stride_bytes, int32_t page_size, int64_t num_pages,
                                               void* kv_a_out, int64_t kv_a_out_stride, void* k_pe_out,
                                               int64_t k_pe_out_stride, const void* q, int64_t q_stride_t,
                                               int64_t q_stride_h, int32_t num_heads, void* q_out, int64_t q_out_stride_t,
                                               int64_t q_out_stride_h, hipStream_t stream) {
  RopeParams qp;
  if (int rc = rope_params("mla_kv_rmsnorm_rope_cache_q_fp8", q, q_stride_t, q_stride_h, num_tokens, num_heads, cos, sin,
                           cs_stride, cos_step, interleaved_out, q_out, q_out_stride_t, q_out_stride_h, &qp))
    return rc;
  return norm_rope_impl(true, kv_a, kv_a_stride, k_pe, k_pe_stride, gamma, cos, sin, cs_stride, cos_step, interleaved_out,
                        slot_mapping, num_tokens, eps, cache, page_stride_bytes, row_stride_bytes, nullptr, 0, 0, page_size,
                        num_pages, kv_a_out, kv_a_out_stride, k_pe_out, k_pe_out_stride, stream, &qp);
}

extern "C" int mla_rotary_mul(const void* x, int64_t x_stride_t, int64_t x_stride_h, int64_t num_tokens, int32_t num_heads,
                              const void* cos, const void* sin, int64_t cs_stride, int32_t cos_step, void* out,
                              int64_t out_stride_t, int64_t out_stride_h, hipStream_t stream) {
  MLA_REQUIRE(x && out, MLA_ERR_NULL, "mla_rotary_mul: null pointer argument");
  if (int rc = check_tables("mla_rotary_mul", cos, sin, cs_stride, cos_step)) return rc;
  MLA_REQUIRE(num_tokens >= 0 && num_heads >= 1 && num_tokens * num_heads < (1ll << 40), MLA_ERR_SHAPE,
              "mla_rotary_mul: num_tokens=%lld num_heads=%d", (long long)num_tokens, num_heads);
  MLA_REQUIRE(x_stride_t % 4 == 0 && x_stride_h % 4 == 0 && out_stride_t % 4 == 0 && out_stride_h % 4 == 0 &&
                  (uintptr_t)x % 8 == 0 && (uintptr_t)out % 8 == 0,
              MLA_ERR_SHAPE, "mla_rotary_mul: rows must be 8-byte aligned");
  if (num_tokens == 0) return MLA_OK;
  RopeParams p;
  p.x = (const __bf16*)x; p.x_st = x_stride_t; p.x_sh = x_stride_h; p.out = (__bf16*)out; p.o_st = out_stride_t;
  p.o_sh = out_stride_h; p.cos = (const __bf16*)cos; p.sin = (const __bf16*)sin; p.cs_stride = cs_stride;
  p.cos_step = cos_step; p.num_tokens = num_tokens; p.num_heads = num_heads; p.interleaved_out = 0;
  const int64_t threads = num_tokens * num_heads * 8;
  hipLaunchKernelGGL(rotary_mul_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, p);
  return check_launch("mla_rotary_mul");
}
