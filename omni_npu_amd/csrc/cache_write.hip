// Latent-KV cache write: row scatter of the new tokens' compressed KV into the paged caches.
//
// Replaces npu_scatter_nd_update_ as used by store_kv in
// src/omni_npu/attention/backends/mla.py:868-881 (and dsa.py:359-362, indexer K at
// vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:116-121):
//   cache.flatten(0, 1)[slot[t], :] = src[t, :],   slot = page * page_size + offset,
// skipping negative (padding) slots and slots past the end of the cache.
#include "mla_common.hpp"

namespace mlahip {

struct ScatterSrc {
  const char* src; int64_t src_stride_b;           // bytes between source rows
  char* cache; int64_t page_stride_b, row_stride_b;
  int32_t row_bytes;                                // multiple of 16
};

// One wavefront per (token, source): 16 bytes per lane per step.
template <int NSRC>
__global__ __launch_bounds__(256) void scatter_rows_kernel(ScatterSrc s0, ScatterSrc s1, const int64_t* slots,
                                                           int32_t num_tokens, int32_t page_size, int64_t num_pages) {
  const int lane = threadIdx.x & 63;
  const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t t = w / NSRC;
  if (t >= num_tokens) return;
  const ScatterSrc& s = (NSRC == 2 && (w % NSRC) == 1) ? s1 : s0;
  // the slot and the first 1 KiB of the row are asked for together (one memory round trip in front of the store, not two)
  const char* src = s.src + t * s.src_stride_b;
  const int i0 = lane * 16;
  u32x4 first = {0u, 0u, 0u, 0u};
  if (i0 < s.row_bytes) first = *(const u32x4*)(src + i0);
  const int64_t slot = slots[t];
  if (slot < 0 || slot >= num_pages * page_size) return;
  int64_t pg, off;
  if (slot < (1ll << 31)) {                                  // 32-bit division where it is enough (64-bit is a long routine)
    const uint32_t pg32 = (uint32_t)slot / (uint32_t)page_size;
    pg = pg32;
    off = (uint32_t)slot - pg32 * (uint32_t)page_size;
  } else {
    pg = slot / page_size;
    off = slot - pg * page_size;
  }
  char* dst = s.cache + pg * s.page_stride_b + off * s.row_stride_b;
  if (i0 < s.row_bytes) *(u32x4*)(dst + i0) = first;
  for (int i = i0 + 64 * 16; i < s.row_bytes; i += 64 * 16) *(u32x4*)(dst + i) = *(const u32x4*)(src + i);
}

}  // namespace mlahip
using namespace mlahip;

extern "C" int mla_cache_write_bf16(const void* kv_c, int64_t kv_c_stride, const void* k_pe, int64_t k_pe_stride,
                                    const int64_t* slot_mapping, int32_t num_tokens, void* nope_cache,
                                    int64_t nope_page_stride, int64_t nope_row_stride, void* rope_cache,
                                    int64_t rope_page_stride, int64_t rope_row_stride, int32_t page_size,
                                    int64_t num_pages, hipStream_t stream) {
  MLA_REQUIRE(kv_c && k_pe && slot_mapping && nope_cache && rope_cache, MLA_ERR_NULL,
              "mla_cache_write_bf16: null pointer argument");
  MLA_REQUIRE(num_tokens >= 0 && page_size >= 1 && num_pages >= 1, MLA_ERR_SHAPE,
              "mla_cache_write_bf16: num_tokens=%d page_size=%d num_pages=%lld", num_tokens, page_size, (long long)num_pages);
  MLA_REQUIRE(kv_c_stride % 8 == 0 && k_pe_stride % 8 == 0 && nope_row_stride % 8 == 0 && rope_row_stride % 8 == 0 &&
                  nope_page_stride % 8 == 0 && rope_page_stride % 8 == 0 && (uintptr_t)kv_c % 16 == 0 &&
                  (uintptr_t)k_pe % 16 == 0 && (uintptr_t)nope_cache % 16 == 0 && (uintptr_t)rope_cache % 16 == 0,
              MLA_ERR_SHAPE, "mla_cache_write_bf16: rows must be 16-byte aligned");
  if (num_tokens == 0) return MLA_OK;
  ScatterSrc a{(const char*)kv_c, kv_c_stride * 2, (char*)nope_cache, nope_page_stride * 2, nope_row_stride * 2, kDNope * 2};
  ScatterSrc b{(const char*)k_pe, k_pe_stride * 2, (char*)rope_cache, rope_page_stride * 2, rope_row_stride * 2, kDRope * 2};
  const int64_t waves = (int64_t)num_tokens * 2;
  hipLaunchKernelGGL(scatter_rows_kernel<2>, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream, a, b, slot_mapping,
                     num_tokens, page_size, num_pages);
  return check_launch("mla_cache_write_bf16");
}

extern "C" int mla_scatter_rows(const void* src, int64_t src_stride_bytes, int32_t row_bytes, const int64_t* slot_mapping,
                                int32_t num_tokens, void* cache, int64_t page_stride_bytes, int64_t row_stride_bytes,
                                int32_t page_size, int64_t num_pages, hipStream_t stream) {
  MLA_REQUIRE(src && slot_mapping && cache, MLA_ERR_NULL, "mla_scatter_rows: null pointer argument");
  MLA_REQUIRE(num_tokens >= 0 && page_size >= 1 && num_pages >= 1 && row_bytes >= 16, MLA_ERR_SHAPE,
              "mla_scatter_rows: num_tokens=%d page_size=%d num_pages=%lld row_bytes=%d", num_tokens, page_size,
              (long long)num_pages, row_bytes);
  MLA_REQUIRE(row_bytes % 16 == 0 && src_stride_bytes % 16 == 0 && page_stride_bytes % 16 == 0 &&
                  row_stride_bytes % 16 == 0 && (uintptr_t)src % 16 == 0 && (uintptr_t)cache % 16 == 0,
              MLA_ERR_SHAPE, "mla_scatter_rows: rows must be multiples of 16 bytes and 16-byte aligned");
  if (num_tokens == 0) return MLA_OK;
  ScatterSrc a{(const char*)src, src_stride_bytes, (char*)cache, page_stride_bytes, row_stride_bytes, row_bytes};
  hipLaunchKernelGGL(scatter_rows_kernel<1>, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256), 0, stream, a, a,
                     slot_mapping, num_tokens, page_size, num_pages);
  return check_launch("mla_scatter_rows");
}

// ------------------------------------------------------------------------------------------------
// fp8-e4m3 block-scaled latent cache.  One cache row (656 bytes) per token:
//   [0,512)    512 x float8_e4m3fn   latent, quantised per 128-element block
//   [512,528)  4 x fp32              block scales (scale = amax / 448, 1.0 for an all-zero block)
//   [528,656)  64 x bf16             rope part, stored unquantised
// The reference has no fp8 KV format (attention/ops.py:11-12 ignores its scale argument), so this
// layout is this library's own; the arithmetic is the closed form x_q = rne_e4m3(x / scale).
// One wavefront per token: lane l owns latent elements [8l, 8l+8); 16 lanes share a block.
namespace mlahip {
constexpr int kFp8RowB = 656;
constexpr int kFp8ScaleOff = 512;
constexpr int kFp8RopeOff = 528;

__global__ __launch_bounds__(256) void cache_write_fp8_kernel(const __bf16* kv_c, int64_t kv_c_stride, const __bf16* k_pe,
                                                              int64_t k_pe_stride, const int64_t* slots,
                                                              int32_t num_tokens, char* cache, int64_t page_stride_b,
                                                              int64_t row_stride_b, int32_t page_size,
                                                              int64_t num_pages) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= num_tokens) return;
  const int64_t slot = slots[t];
  if (slot < 0 || slot >= num_pages * page_size) return;
  const int64_t pg = slot / page_size;
  char* row = cache + pg * page_stride_b + (slot - pg * page_size) * row_stride_b;

  const bf16x8 v = *(const bf16x8*)(kv_c + t * kv_c_stride + lane * 8);
  float x[8];
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) { x[e] = (float)v[e]; amax = fmaxf(amax, fabsf(x[e])); }
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));   // 16 lanes = one 128-block
  const float scale = amax > 0.f ? amax / 448.f : 1.f;
  float y[8];
#pragma unroll
  for (int e = 0; e < 8; e++) y[e] = fminf(fmaxf(x[e] / scale, -448.f), 448.f);
  int w0 = 0, w1 = 0;
  w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
  w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
  w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
  w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
  u32x2 packed = {(uint32_t)w0, (uint32_t)w1};
  *(u32x2*)(row + lane * 8) = packed;
  if ((lane & 15) == 0) *(float*)(row + kFp8ScaleOff + (lane >> 4) * 4) = scale;
  if (lane < 8) *(u32x4*)(row + kFp8RopeOff + lane * 16) = *(const u32x4*)((const char*)(k_pe + t * k_pe_stride) + lane * 16);
}
}  // namespace mlahip

extern "C" int mla_cache_write_fp8(const void* kv_c, int64_t kv_c_stride, const void* k_pe, int64_t k_pe_stride,
                                   const int64_t* slot_mapping, int32_t num_tokens, void* cache,
                                   int64_t page_stride_bytes, int64_t row_stride_bytes, int32_t page_size,
                                   int64_t num_pages, hipStream_t stream) {
  MLA_REQUIRE(kv_c && k_pe && slot_mapping && cache, MLA_ERR_NULL, "mla_cache_write_fp8: null pointer argument");
  MLA_REQUIRE(num_tokens >= 0 && page_size >= 1 && num_pages >= 1, MLA_ERR_SHAPE,
              "mla_cache_write_fp8: num_tokens=%d page_size=%d num_pages=%lld", num_tokens, page_size, (long long)num_pages);
  MLA_REQUIRE(row_stride_bytes >= kFp8RowB && row_stride_bytes % 16 == 0 && page_stride_bytes % 16 == 0 &&
                  kv_c_stride % 8 == 0 && k_pe_stride % 8 == 0 && (uintptr_t)kv_c % 16 == 0 && (uintptr_t)k_pe % 16 == 0 &&
                  (uintptr_t)cache % 16 == 0,
              MLA_ERR_SHAPE, "mla_cache_write_fp8: rows are 656 bytes, 16-byte aligned");
  if (num_tokens == 0) return MLA_OK;
  hipLaunchKernelGGL(cache_write_fp8_kernel, dim3((unsigned)((num_tokens + 3) / 4)), dim3(256), 0, stream,
                     (const __bf16*)kv_c, kv_c_stride, (const __bf16*)k_pe, k_pe_stride, slot_mapping, num_tokens,
                     (char*)cache, page_stride_bytes, row_stride_bytes, page_size, num_pages);
  return check_launch("mla_cache_write_fp8");
}
