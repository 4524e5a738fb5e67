// Host entry points of the absorbed-MLA paged decode (C-ABI): argument checks, workspace layout, launches.
//
// Replaces the reference's decode call of npu_fused_infer_attention_score
// (src/omni_npu/attention/backends/mla.py:781-804): for sequence b, head n, query token t
//   s_j = scale * (ql[t,n] . Kc[j] + qr[t,n] . Kr[j]),  j < L_b - (q_len-1-t)   (right-down causal)
//   o   = sum_j softmax(s)_j * Kc[j]
// with ONE latent KV row (512 + 64) shared by all heads.  The kernels live in decode_v3.hip (bf16 cache: dense, row-list
// and sink + window sources), decode_v3_fp8.hip (fp8-e4m3 block-scaled cache) and chunk_reduce.hip (the merge of the
// split-KV partials: the N-way merge of src/omni_npu/attention/ops.py:109-141).
//
// Workspace (mla_decode_workspace_bytes): batch * (num_splits + 1) partial slots of rows = max_q_len * num_heads each:
// normalised fp16 partials [slots, rows, 512], fp32 log-sum-exps [slots, rows], a correction record per row (fp32
// factor + cache address of the row's dominant key) and two partial numbers per sequence.
#include <cstdlib>
#include <mutex>
#include "mla_common.hpp"
#include "decode_params.hpp"

namespace mlahip {
constexpr int kRowsPerWg = 128;
constexpr int kFp8RowB = 656;
}  // namespace mlahip

using namespace mlahip;

extern "C" size_t mla_decode_workspace_bytes(int32_t batch, int32_t max_q_len, int32_t num_heads, int32_t num_splits) {
  if (batch <= 0 || max_q_len <= 0 || num_heads <= 0 || num_splits <= 0) return 0;
  // batch * num_splits chunks, and one more partial for every sequence boundary inside a chunk: batch * (num_splits + 1) partials in all
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * max_q_len * num_heads;
  // fp16 partials, fp32 log-sum-exps, and per row a correction record (fp32 factor + cache address)
  // ... and two partial numbers per sequence
  return rows * kDNope * sizeof(_Float16) + rows * (2 * sizeof(float) + sizeof(void*)) + (size_t)batch * 2 * sizeof(int32_t);
}

static int decode_split_impl(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                     int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                     int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                     int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                     const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                     const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                     int32_t max_q_len, int32_t num_heads, float scale, void* workspace,
                                     size_t workspace_bytes, int32_t num_splits, const int32_t* sparse_rows,
                                     int64_t sparse_stride, int32_t page_size, bool fp8, hipStream_t stream,
                                     const int32_t* win_skip = nullptr, int32_t win_sink = 0, int32_t win_size = 0,
                                     const void* new_c = nullptr, int64_t new_c_stride = 0, const void* new_r = nullptr,
                                     int64_t new_r_stride = 0, const int64_t* new_slots = nullptr) {
  MLA_REQUIRE(q_nope && q_rope && nope_cache && rope_cache && (block_table || sparse_rows) && seq_lens, MLA_ERR_NULL,
              "mla_decode_bf16: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_splits >= 1 && (sparse_rows || max_blocks >= 1) &&
                  num_pages >= 1 && page_size >= 1,
              MLA_ERR_SHAPE, "mla_decode_bf16: batch=%d max_q_len=%d num_heads=%d num_splits=%d max_blocks=%d num_pages=%lld",
              batch, max_q_len, num_heads, num_splits, max_blocks, (long long)num_pages);
  MLA_REQUIRE(num_splits <= 65535 && batch <= 65535, MLA_ERR_SHAPE, "mla_decode_bf16: grid limits exceeded");
  MLA_REQUIRE((qn_stride_t % 8 == 0) && (qn_stride_h % 8 == 0) && (qr_stride_t % 8 == 0) && (qr_stride_h % 8 == 0) &&
                  (nope_row_stride % 8 == 0) && (rope_row_stride % 8 == 0) && (nope_page_stride % 8 == 0) &&
                  (rope_page_stride % 8 == 0),
              MLA_ERR_SHAPE, "mla_decode_bf16: strides must keep 16-byte alignment of 8-element groups");
  MLA_REQUIRE(((uintptr_t)q_nope % 16 == 0) && ((uintptr_t)q_rope % 16 == 0) && ((uintptr_t)nope_cache % 16 == 0) &&
                  ((uintptr_t)rope_cache % 16 == 0),
              MLA_ERR_SHAPE, "mla_decode_bf16: pointers must be 16-byte aligned");
  if (batch == 0) return MLA_OK;
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(workspace && workspace_bytes >= need, MLA_ERR_WORKSPACE,
              "mla_decode_bf16: workspace %zu bytes < required %zu", workspace_bytes, need);
  MLA_REQUIRE((uintptr_t)workspace % 16 == 0, MLA_ERR_SHAPE, "mla_decode_bf16: workspace must be 16-byte aligned");

  const int r_max = max_q_len * num_heads;
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * r_max;
  MLA_REQUIRE((int64_t)batch * num_splits <= 0x7fffffff / 2 && nope_row_stride < (1 << 28) && rope_row_stride < (1 << 28),
              MLA_ERR_SHAPE, "mla_decode_bf16: batch * num_splits or a row stride is out of range");
  DecodeParams v;
  v.q_nope = (const __bf16*)q_nope; v.qn_st = qn_stride_t; v.qn_sh = qn_stride_h;
  v.q_rope = (const __bf16*)q_rope; v.qr_st = qr_stride_t; v.qr_sh = qr_stride_h;
  v.nope = (const __bf16*)nope_cache; v.nope_sp = nope_page_stride; v.nope_sr = nope_row_stride;
  v.rope = (const __bf16*)rope_cache; v.rope_sp = rope_page_stride; v.rope_sr = rope_row_stride;
  v.block_table = block_table; v.bt_stride = bt_stride; v.max_blocks = max_blocks;
  v.seq_lens = seq_lens; v.qsl = query_start_loc;
  v.batch = batch; v.max_q_len = max_q_len; v.num_heads = num_heads; v.num_pages = num_pages;
  v.scale_log2 = scale * kLog2e;
  v.o_part = (_Float16*)workspace;
  v.lse_part = (float*)((_Float16*)workspace + rows * kDNope);
  v.corr_scale = v.lse_part + rows; v.corr_row = (const __bf16**)(v.lse_part + 2 * rows);
  v.seg_ids = (int32_t*)(v.lse_part + 4 * rows);
  v.sparse_rows = sparse_rows; v.sparse_stride = sparse_stride; v.page_size = page_size;
  v.cache8 = fp8 ? (const uint8_t*)nope_cache : nullptr; v.c8_sp = nope_page_stride;
  v.win_skip = win_skip; v.win_sink = win_sink; v.win_size = win_size;
  v.new_c = (const __bf16*)new_c; v.new_c_st = new_c_stride; v.new_r = (const __bf16*)new_r; v.new_r_st = new_r_stride;
  v.new_slots = new_slots;
  // one workgroup per (balanced chunk, group of 128 query rows)
  const dim3 grid((unsigned)(batch * num_splits), 1, (unsigned)((r_max + kRowsPerWg - 1) / kRowsPerWg));
  if (fp8) return launch_decode_v3_fp8(v, grid, stream);
  return launch_decode_v3(v, sparse_rows != nullptr, grid, stream);
}

// Phase 1: one normalised fp16 partial + log-sum-exp per (segment of a chunk, query row) into the workspace.
extern "C" int mla_decode_bf16_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                     int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                     int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                     int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                     const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                     const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                     int32_t max_q_len, int32_t num_heads, float scale, void* workspace,
                                     size_t workspace_bytes, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(block_table, MLA_ERR_NULL, "mla_decode_bf16: null block table");
  return decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                           nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                           block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads,
                           scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, false, stream);
}

// Static sink tokens + sliding window on the dense kernel.  mla_window_plan turns the lengths behind the sink into the
// lengths of the shortened sequences the kernel walks (sink keys + the blocks that hold some token's window) and the
// number of 32-key blocks left out; mla_decode_bf16_window_split is mla_decode_bf16_split over those, and the merge is
// the ordinary one with the shortened lengths.
namespace mlahip {
__global__ void mla_window_plan_kernel(const int32_t* seq_lens, const int32_t* qsl, int32_t batch, int32_t max_q_len,
                                       int32_t sink_len, int32_t window, int32_t* short_lens, int32_t* skip) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  int qlen = qsl ? qsl[b + 1] - qsl[b] : max_q_len;
  qlen = qlen < max_q_len ? qlen : max_q_len;
  const int len = seq_lens[b];
  int n0 = len - qlen + 1;                                   // keys the request's first query token sees
  n0 = n0 < 0 ? 0 : n0;
  const int lo0 = n0 > window ? n0 - window : 0;             // the oldest key any of its tokens sees
  const int sk = lo0 / 32;
  skip[b] = sk;
  short_lens[b] = len > 0 ? sink_len + len - sk * 32 : 0;
}
}  // namespace mlahip

extern "C" int mla_window_plan(const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch, int32_t max_q_len,
                               int32_t sink_len, int32_t window, int32_t* short_lens, int32_t* skip, hipStream_t stream) {
  MLA_REQUIRE(seq_lens && short_lens && skip, MLA_ERR_NULL, "mla_window_plan: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && sink_len >= 0 && sink_len % kPage == 0 && window >= 1, MLA_ERR_SHAPE,
              "mla_window_plan: batch=%d max_q_len=%d sink_len=%d window=%d", batch, max_q_len, sink_len, window);
  if (batch == 0) return MLA_OK;
  hipLaunchKernelGGL(mla_window_plan_kernel, dim3((batch + 255) / 256), dim3(256), 0, stream, seq_lens, query_start_loc, batch,
                     max_q_len, sink_len, window, short_lens, skip);
  return check_launch("mla_window_plan_kernel");
}

extern "C" int mla_decode_bf16_window_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                            int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                            int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                            int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                            const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                            const int32_t* short_lens, const int32_t* skip, const int32_t* query_start_loc,
                                            int32_t batch, int32_t max_q_len, int32_t num_heads, int32_t sink_len,
                                            int32_t window, float scale, void* workspace, size_t workspace_bytes,
                                            int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(block_table && skip, MLA_ERR_NULL, "mla_decode_bf16_window_split: null block table or skip counts");
  MLA_REQUIRE(sink_len >= 0 && sink_len % kPage == 0 && window >= 1, MLA_ERR_SHAPE,
              "mla_decode_bf16_window_split: sink_len=%d window=%d", sink_len, window);
  return decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                           nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                           block_table, bt_stride, max_blocks, short_lens, query_start_loc, batch, max_q_len, num_heads,
                           scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, false, stream, skip, sink_len,
                           window);
}

// The windowed split phase over the fp8 block-scaled cache (same plan, same merge).
extern "C" int mla_decode_fp8_window_split(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                           int64_t qr_stride_t, int64_t qr_stride_h, const void* cache, int64_t page_stride_bytes,
                                           int64_t row_stride_bytes, int64_t num_pages, const int32_t* block_table,
                                           int64_t bt_stride, int32_t max_blocks, const int32_t* short_lens, const int32_t* skip,
                                           const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                           int32_t sink_len, int32_t window, float scale, void* workspace,
                                           size_t workspace_bytes, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(cache && block_table && skip, MLA_ERR_NULL, "mla_decode_fp8_window_split: null pointer argument");
  MLA_REQUIRE(row_stride_bytes == kFp8RowB && page_stride_bytes >= (int64_t)kPage * kFp8RowB && page_stride_bytes % 16 == 0,
              MLA_ERR_UNSUPPORTED, "mla_decode_fp8_window_split: rows must be exactly 656 bytes apart, pages 128 rows (got %lld / %lld)",
              (long long)row_stride_bytes, (long long)page_stride_bytes);
  MLA_REQUIRE(sink_len >= 0 && sink_len % kPage == 0 && window >= 1, MLA_ERR_SHAPE,
              "mla_decode_fp8_window_split: sink_len=%d window=%d", sink_len, window);
  return decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, cache, page_stride_bytes,
                           kFp8RowB + 8, cache, page_stride_bytes, kFp8RowB + 8, num_pages, block_table, bt_stride, max_blocks,
                           short_lens, query_start_loc, batch, max_q_len, num_heads, scale, workspace, workspace_bytes,
                           num_splits, nullptr, 0, kPage, true, stream, skip, sink_len, window);
}

// Phase 2: N-way log-sum-exp merge of the workspace partials into the bf16 output (and optional lse).
extern "C" int mla_splitkv_reduce(const void* workspace, size_t workspace_bytes, const int32_t* seq_lens,
                                  const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t num_heads,
                                  int32_t num_splits, void* out, int64_t out_stride_t, int64_t out_stride_h,
                                  float* lse_out, hipStream_t stream) {
  MLA_REQUIRE(workspace && out && seq_lens, MLA_ERR_NULL, "mla_splitkv_reduce: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_splits >= 1, MLA_ERR_SHAPE,
              "mla_splitkv_reduce: batch=%d max_q_len=%d num_heads=%d num_splits=%d", batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE((out_stride_t % 8 == 0) && (out_stride_h % 8 == 0) && ((uintptr_t)out % 16 == 0) &&
                  ((uintptr_t)workspace % 16 == 0),
              MLA_ERR_SHAPE, "mla_splitkv_reduce: output rows must be 16-byte aligned");
  if (batch == 0) return MLA_OK;
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(workspace_bytes >= need, MLA_ERR_WORKSPACE, "mla_splitkv_reduce: workspace %zu bytes < required %zu",
              workspace_bytes, need);
  const int r_max = max_q_len * num_heads;
  const size_t rows = (size_t)batch * ((size_t)num_splits + 1) * r_max;
  // partials in chunk order, as the split kernels write them
  ChunkReduceParams cp;
  cp.o_part = (const _Float16*)workspace; cp.lse_part = (const float*)((const _Float16*)workspace + rows * kDNope);
  cp.corr_scale = cp.lse_part + rows; cp.corr_row = (const __bf16* const*)(cp.lse_part + 2 * rows);
  cp.seg_ids = (const int32_t*)(cp.lse_part + 4 * rows);
  cp.seq_lens = seq_lens; cp.qsl = query_start_loc;
  cp.batch = batch; cp.max_q_len = max_q_len; cp.num_heads = num_heads; cp.num_chunks = batch * num_splits;
  cp.out = (__bf16*)out; cp.out_st = out_stride_t; cp.out_sh = out_stride_h;
  cp.lse_out = lse_out; cp.lse_st = num_heads;
  return launch_chunk_reduce(cp, stream);
}

// A whole decode step in two launches: the cache write of the step's new tokens (the reshape-and-cache in front of the
// reference's decode, src/omni_npu/attention/backends/mla.py:868-881) rides in the split kernel, then the merge.  Token t
// of the batch (query_start_loc order, or b * max_q_len + j) brings latent row new_c[t] and rope row new_r[t] for cache row
// slot_mapping[t]; negative slots are skipped.  The row of key position p of sequence b is stored by the workgroup
// whose chunk holds p, before that workgroup reads any key, so the result equals mla_cache_write_bf16 followed by
// mla_decode_bf16 for every sequence whose seq_lens counts its new tokens (the rows of a request with fewer cached keys
// than query tokens, e.g. an empty padding request, are not written).  With out == NULL only the first launch runs and
// the partials stay in the workspace for mla_splitkv_reduce.
extern "C" int mla_decode_bf16_step(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                    int64_t qr_stride_t, int64_t qr_stride_h, void* nope_cache, int64_t nope_page_stride,
                                    int64_t nope_row_stride, void* rope_cache, int64_t rope_page_stride,
                                    int64_t rope_row_stride, int64_t num_pages, const void* new_c, int64_t new_c_stride,
                                    const void* new_r, int64_t new_r_stride, const int64_t* slot_mapping,
                                    const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                    const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                    int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                                    int64_t out_stride_h, float* lse_out, void* workspace, size_t workspace_bytes,
                                    int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(block_table && new_c && new_r && slot_mapping, MLA_ERR_NULL, "mla_decode_bf16_step: null pointer argument");
  MLA_REQUIRE(new_c_stride % 8 == 0 && new_r_stride % 8 == 0 && (uintptr_t)new_c % 16 == 0 && (uintptr_t)new_r % 16 == 0,
              MLA_ERR_SHAPE, "mla_decode_bf16_step: the new rows must be 16-byte aligned");
  int rc = decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                             nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                             block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads,
                             scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, false, stream, nullptr, 0, 0,
                             new_c, new_c_stride, new_r, new_r_stride, slot_mapping);
  if (rc != MLA_OK || out == nullptr) return rc;              // (out == NULL: the first launch only, partials in the workspace)
  return mla_splitkv_reduce(workspace, workspace_bytes, seq_lens, query_start_loc, batch, max_q_len, num_heads, num_splits,
                            out, out_stride_t, out_stride_h, lse_out, stream);
}

// Both phases on one stream.
extern "C" int mla_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                               int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                               int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                               int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                               const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                               const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                               int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                               int64_t out_stride_h, float* lse_out, void* workspace, size_t workspace_bytes,
                               int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(out, MLA_ERR_NULL, "mla_decode_bf16: null output pointer");
  int rc = mla_decode_bf16_split(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                                 nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride,
                                 num_pages, block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch,
                                 max_q_len, num_heads, scale, workspace, workspace_bytes, num_splits, stream);
  if (rc != MLA_OK) return rc;
  return mla_splitkv_reduce(workspace, workspace_bytes, seq_lens, query_start_loc, batch, max_q_len, num_heads, num_splits,
                            out, out_stride_t, out_stride_h, lse_out, stream);
}

// The same decode for callers that cannot allocate or hand over a workspace (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the split-KV partials live in a file-scope device array of kStaticScratchBytes.
// Every GPU the library runs on holds its own copy of the array at its own address for the life of the process; the
// address is looked up once per device (hipGetSymbolAddress) and from then on only that pointer is used.  Calls that
// overlap in time on one GPU share the array and race; calls on one stream, or ordered by events, do not.  Nothing has
// to start at zero: the split phase writes every partial, log-sum-exp, correction record and segment number the merge
// reads (the merge derives which ones exist from seq_lens, as the split does).
namespace mlahip {
constexpr size_t kStaticScratchBytes = (size_t)48 << 20;   // 48 MiB: the headline step (64 x 128 heads, 4 splits) needs 42.6 MB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];                    // per device, nullptr = not looked up yet
static std::mutex g_scratch_mutex;

static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(MLA_ERR_LAUNCH, "mla_decode_bf16_static: no current device (hipGetDevice gave %d)", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(MLA_ERR_LAUNCH, "mla_decode_bf16_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    // (every form the entry point may pick later gets its LDS limit now: a later call under capture then only launches)
    const int rc = prepare_decode_v3_dense_forms();
    if (rc != MLA_OK) return rc;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MLA_OK;
}
}  // namespace mlahip

extern "C" int mla_decode_bf16_static(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                      int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                      int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                      int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                      const int32_t* block_table, int64_t bt_stride, int32_t max_blocks,
                                      const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                                      int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                                      int64_t out_stride_h, float* lse_out, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && num_heads >= 1 && num_splits >= 1, MLA_ERR_SHAPE,
              "mla_decode_bf16_static: batch=%d max_q_len=%d num_heads=%d num_splits=%d", batch, max_q_len, num_heads, num_splits);
  const size_t need = mla_decode_workspace_bytes(batch, max_q_len, num_heads, num_splits);
  MLA_REQUIRE(need <= kStaticScratchBytes, MLA_ERR_WORKSPACE,
              "mla_decode_bf16_static: this shape needs %zu bytes of split-KV scratch, the built-in array holds %zu; "
              "use mla_decode_bf16 with a caller-owned workspace", need, (size_t)kStaticScratchBytes);
  void* ptr = nullptr;
  const int rc = static_scratch(&ptr);
  if (rc != MLA_OK) return rc;
  return mla_decode_bf16(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache, nope_page_stride,
                         nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages, block_table, bt_stride,
                         max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads, scale, out, out_stride_t,
                         out_stride_h, lse_out, ptr, kStaticScratchBytes, num_splits, stream);
}

// Sparse absorbed MLA over a per-token list of cache rows (reference: npu_sparse_flash_attention as called in
// src/omni_npu/attention/backends/dsa.py:259-291).  Token t attends to the rows sparse_rows[t, 0 .. counts[t]) that
// dsa_build_rows produced from the indexer's top-k positions.  Same split-KV kernel and reduction as the dense decode.
extern "C" int dsa_sparse_decode_bf16(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                                      int64_t qr_stride_t, int64_t qr_stride_h, const void* nope_cache,
                                      int64_t nope_page_stride, int64_t nope_row_stride, const void* rope_cache,
                                      int64_t rope_page_stride, int64_t rope_row_stride, int64_t num_pages,
                                      int32_t page_size, const int32_t* sparse_rows, int64_t sparse_stride,
                                      const int32_t* counts, int32_t num_tokens, int32_t num_heads, float scale, void* out,
                                      int64_t out_stride_t, int64_t out_stride_h, float* lse_out, void* workspace,
                                      size_t workspace_bytes, int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(sparse_rows && counts, MLA_ERR_NULL, "dsa_sparse_decode_bf16: null pointer argument");
  MLA_REQUIRE(sparse_stride >= 1 && page_size >= 1, MLA_ERR_SHAPE, "dsa_sparse_decode_bf16: sparse_stride=%lld page_size=%d",
              (long long)sparse_stride, page_size);
  MLA_REQUIRE(nope_page_stride == (int64_t)page_size * nope_row_stride && rope_page_stride == (int64_t)page_size * rope_row_stride,
              MLA_ERR_UNSUPPORTED, "dsa_sparse_decode_bf16: cache pages must be contiguous (page stride == page_size * row stride)");
  int rc = decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, nope_cache,
                             nope_page_stride, nope_row_stride, rope_cache, rope_page_stride, rope_row_stride, num_pages,
                             nullptr, 0, 0, counts, nullptr, num_tokens, 1, num_heads, scale, workspace, workspace_bytes,
                             num_splits, sparse_rows, sparse_stride, page_size, false, stream);
  if (rc != MLA_OK || !out) return rc;                      // out == NULL: split phase only, the partials stay in the workspace
  return mla_splitkv_reduce(workspace, workspace_bytes, counts, nullptr, num_tokens, 1, num_heads, num_splits, out,
                            out_stride_t, out_stride_h, lse_out, stream);
}

// Absorbed-MLA paged decode over the fp8-e4m3 block-scaled cache written by mla_cache_write_fp8 (656-byte rows,
// row stride exactly 656, page size 128).  Tiles are dequantised to bf16 in LDS and then take the bf16 MFMA path, so
// the arithmetic is "dequantise, then attend" as in the CPU restatement.  The reference has no fp8 cache
// (src/omni_npu/attention/backends/mla.py:791-792 passes antiquant_mode=0, antiquant_scale=None).
extern "C" int mla_decode_fp8(const void* q_nope, int64_t qn_stride_t, int64_t qn_stride_h, const void* q_rope,
                              int64_t qr_stride_t, int64_t qr_stride_h, const void* cache, int64_t page_stride_bytes,
                              int64_t row_stride_bytes, int64_t num_pages, const int32_t* block_table, int64_t bt_stride,
                              int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                              int32_t max_q_len, int32_t num_heads, float scale, void* out, int64_t out_stride_t,
                              int64_t out_stride_h, float* lse_out, void* workspace, size_t workspace_bytes,
                              int32_t num_splits, hipStream_t stream) {
  MLA_REQUIRE(cache && block_table, MLA_ERR_NULL, "mla_decode_fp8: null pointer argument");
  MLA_REQUIRE(row_stride_bytes == kFp8RowB && page_stride_bytes >= (int64_t)kPage * kFp8RowB && page_stride_bytes % 16 == 0,
              MLA_ERR_UNSUPPORTED, "mla_decode_fp8: rows must be exactly 656 bytes apart, pages 128 rows (got %lld / %lld)",
              (long long)row_stride_bytes, (long long)page_stride_bytes);
  // the shared validation wants element strides that are multiples of 8: hand it byte strides that are
  int rc = decode_split_impl(q_nope, qn_stride_t, qn_stride_h, q_rope, qr_stride_t, qr_stride_h, cache, page_stride_bytes,
                             kFp8RowB + 8 /* unused in fp8 mode */, cache, page_stride_bytes, kFp8RowB + 8, num_pages,
                             block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len, num_heads,
                             scale, workspace, workspace_bytes, num_splits, nullptr, 0, kPage, true, stream);
  if (rc != MLA_OK || !out) return rc;                      // out == NULL: split phase only, the partials stay in the workspace
  // partials come in the balanced chunk order of the bf16 path: the same merge
  return mla_splitkv_reduce(workspace, workspace_bytes, seq_lens, query_start_loc, batch,
                            max_q_len, num_heads, num_splits, out, out_stride_t, out_stride_h, lse_out, stream);
}
