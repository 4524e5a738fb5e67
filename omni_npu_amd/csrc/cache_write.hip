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
  const int64_t slot = slots[t];
  if (slot < 0 || slot >= num_pages * page_size) return;
  const int64_t pg = slot / page_size;
  const int64_t off = slot - pg * page_size;
  const char* src = s.src + t * s.src_stride_b;
  char* dst = s.cache + pg * s.page_stride_b + off * s.row_stride_b;
  for (int i = lane * 16; i < s.row_bytes; i += 64 * 16) *(u32x4*)(dst + i) = *(const u32x4*)(src + i);
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
