// Exact top-k selection for the DSA indexer, and the index -> cache-row translation for sparse MLA.
//
// Replaces the selection half of torch.ops.custom.npu_lightning_indexer
// (src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:133-146: int32 [T,1,topk]
// logical key positions, -1 for unused slots as in src/omni_npu/v1/layers/attention/npu_dsa.py:553-555).
// Semantics: the k largest logits among the visible keys, ties to the LOWER index; the output lists the
// selected positions in ascending position order followed by -1 padding.
//
// One workgroup of 1024 threads per query token, three coalesced sweeps over the row (it stays in L2):
//   1. histogram over 2048 bins that are linear in the (sampled) range of the logits, which names the bin holding the
//      k-th largest logit;
//   2. the keys of that bin (a few dozen for a smooth distribution) move to LDS, where the exact threshold is found on
//      the 64-bit key  (order-preserving image of the fp32 logit) << 32 | ~position  (all keys are distinct, so
//      "key >= threshold" selects exactly k elements) - by ranking when they are few, by a radix select otherwise -
//      while every wavefront counts the sure picks of its contiguous range;
//   3. the selected positions are written in order with ballot prefix sums.
#include "mla_common.hpp"

namespace mlahip {

constexpr int kTopkThreads = 1024;
constexpr int kBins = 2048;

__device__ __forceinline__ uint32_t ordered_bits(float x) {
  if (x == 0.f) x = 0.f;                                   // -0 and +0 compare equal: one image for both
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Workgroup-wide: given hist[kBins] (count per digit, larger digit = larger key) and `need` (>= 1, <= total),
// find digit d with  count(digit > d) < need <= count(digit >= d).  Returns d, and the count above it via *above.
__device__ int select_digit(int* hist, int* scratch, int need, int* above) {
  const int tid = threadIdx.x;
  // each thread owns 2 bins taken from the top: bins (kBins-1-2*tid) and (kBins-2-2*tid)
  const int b0 = kBins - 1 - 2 * tid, b1 = b0 - 1;
  const int c0 = hist[b0], c1 = hist[b1];
  int v = c0 + c1;
  // inclusive scan over threads (descending bins)
  const int lane = tid & 63, w = tid >> 6;
  int s = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int n = __shfl_up(s, o, 64);
    if (lane >= o) s += n;
  }
  if (lane == 63) scratch[w] = s;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += scratch[i];
  const int incl = base + s, excl = incl - v;              // keys in bins above this thread's pair: excl
  __syncthreads();
  if (excl < need && need <= incl) {                       // exactly one thread
    if (need <= excl + c0) { scratch[32] = b0; scratch[33] = excl; }
    else { scratch[32] = b1; scratch[33] = excl + c0; }
  }
  __syncthreads();
  const int d = scratch[32];
  *above = scratch[33];
  __syncthreads();
  return d;
}

struct TopkParams {
  const float* logits; int64_t l_st;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, k;
  int32_t* out; int64_t o_st;
  // optional (rows != NULL): also translate every pick into its flat cache row, and count the picks per token
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks, page_size; int64_t num_pages;
  int32_t* rows; int64_t r_st; int32_t* counts;
};

// Where pick number `at` of token t (request b) goes: its position into the index buffer and, if asked for, its flat
// cache row (page * page_size + offset) into the row list that the sparse attention reads.
struct TopkSink {
  int32_t* out; int32_t* rows; const int32_t* bt; int32_t max_blocks, page_size; int64_t num_pages;
  __device__ __forceinline__ void put(int at, int pos) const {
    out[at] = pos;
    if (rows) {
      int pg = pos / page_size;
      const int off = pos - pg * page_size;
      pg = pg < max_blocks ? pg : max_blocks - 1;
      int64_t blk = bt[pg];
      blk = blk < 0 ? 0 : (blk >= num_pages ? num_pages - 1 : blk);
      rows[at] = (int32_t)(blk * page_size + off);
    }
  }
};
__device__ __forceinline__ TopkSink topk_sink(const TopkParams& p, int b, int t) {
  TopkSink s;
  s.out = p.out + (int64_t)t * p.o_st;
  s.rows = p.rows ? p.rows + (int64_t)t * p.r_st : nullptr;
  s.bt = p.rows ? p.block_table + (int64_t)b * p.bt_stride : nullptr;
  s.max_blocks = p.max_blocks; s.page_size = p.page_size; s.num_pages = p.num_pages;
  return s;
}

constexpr int kCandCap = 8192;                             // boundary-bin keys that fit in LDS
constexpr int kRankMax = 256;                              // up to here the threshold is found by ranking, not by radix passes

// Monotone map of a logit to one of kBins bins, linear over [lo, hi] and clamped outside: x <= y implies
// bin(x) <= bin(y) (every step - fused multiply-add, conversion, clamp - is monotone) for ANY scale >= 0 and shift, so
// the range only has to be roughly right; NaNs go where their ordered image puts them.  A radix digit of the float's
// bit pattern would pile almost every key of a smooth distribution into a handful of bins (same exponent), and LDS
// atomics on one address serialise.
__device__ __forceinline__ int linear_bin(float x, float scale, float shift) {
  if (x != x) return (__float_as_uint(x) & 0x80000000u) ? 0 : kBins - 1;
  const int b = (int)__builtin_fmaf(x, scale, shift);      // saturating conversion
  return b < 0 ? 0 : (b > kBins - 1 ? kBins - 1 : b);
}

// f(value, position) for every key of [lo, hi), `group` threads side by side (`me` = this thread's number in the
// group), kVec consecutive keys per thread and load, eight loads in flight
// (the row comes from L2 / HBM at most of a microsecond a round trip: a loop that uses each value before asking for the
// next is latency bound).  With kVec = 4 the row must be 16-byte
// aligned and lo a multiple of 4.  Keys are visited in ascending position within a thread.
template <int kVec, class F>
__device__ __forceinline__ void sweep(const float* x, int lo, int hi, int me, int group, F f) {
  constexpr int kDepth = 8;
  for (int c0 = lo + me * kVec; c0 < hi; c0 += group * kVec * kDepth) {
    float v[kDepth][kVec];
#pragma unroll
    for (int j = 0; j < kDepth; j++) {
      const int i = c0 + j * group * kVec;
      if (kVec == 4) {
        if (i + 3 < hi) {
          const f32x4 q = *(const f32x4*)(x + i);
          v[j][0] = q[0]; v[j][1] = q[1]; v[j][2] = q[2]; v[j][3] = q[3];
        } else {
#pragma unroll
          for (int e = 0; e < kVec; e++) v[j][e] = i + e < hi ? x[i + e] : 0.f;
        }
      } else {
        v[j][0] = i < hi ? x[i] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < kDepth; j++)
#pragma unroll
      for (int e = 0; e < kVec; e++) {
        const int i = c0 + j * group * kVec + e;
        if (i < hi) f(v[j][e], i);
      }
  }
}

// Exact threshold among the keys that `each` enumerates (callback(u, pos) for every key of the set): returns the image
// `prefix` of the threshold logit and the highest position still taken among the keys equal to it, such that exactly
// `need` keys of the set satisfy  u > prefix || (u == prefix && pos <= pos_thresh).  Radix select over the 64-bit key
// (u << 32 | ~pos): three 11/11/10-bit passes over u, two 11-bit passes over ~pos.
template <int kThreads, class Each>
__device__ void radix_threshold(Each each, int need, int* hist, int* scratch, uint32_t* prefix_out, uint32_t* pos_out) {
  const int tid = threadIdx.x;
  uint32_t prefix = 0, pmask = 0;
  const int shifts[3] = {21, 10, 0};
  const int widths[3] = {11, 11, 10};
  for (int pass = 0; pass < 3; pass++) {
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    const int sh = shifts[pass];
    const uint32_t dm = (1u << widths[pass]) - 1;
    each([&](uint32_t u, uint32_t) {
      if ((u & pmask) == prefix) atomicAdd(&hist[(u >> sh) & dm], 1);
    });
    __syncthreads();
    int above;
    const int d = select_digit(hist, scratch, need, &above);
    need -= above;
    prefix |= (uint32_t)d << sh;
    pmask |= dm << sh;
  }
  // `need` (>= 1) of the keys equal to the threshold are wanted: the lowest positions among them
  uint32_t ppre = 0, pm = 0;
  const int psh[2] = {11, 0};
  for (int pass = 0; pass < 2; pass++) {
    for (int i = tid; i < kBins; i += kThreads) hist[i] = 0;
    __syncthreads();
    each([&](uint32_t u, uint32_t pos) {
      if (u == prefix) {
        const uint32_t ip = (~pos) & 0x3FFFFFu;            // larger digit of ~pos = lower position
        if ((ip & pm) == ppre) atomicAdd(&hist[(ip >> psh[pass]) & 0x7FFu], 1);
      }
    });
    __syncthreads();
    int above;
    const int d = select_digit(hist, scratch, need, &above);
    need -= above;
    ppre |= (uint32_t)d << psh[pass];
    pm |= 0x7FFu << psh[pass];
  }
  *prefix_out = prefix;
  *pos_out = (~ppre) & 0x3FFFFFu;
}

// Threshold among m <= kRankMax candidates in LDS by ranking: the candidate with exactly `need - 1` larger keys.  All
// 1024 threads take part: thread (c, g) compares candidate c with candidates g, g + G, ... and the partial ranks meet in
// `rank` (LDS, at least kRankMax ints).
__device__ __forceinline__ void rank_threshold(const uint32_t* cand_u, const uint32_t* cand_i, int m, int need, int* rank,
                                               int* scratch, uint32_t* prefix_out, uint32_t* pos_out) {
  const int tid = threadIdx.x;
  int mpad = 64;
  while (mpad < m) mpad <<= 1;
  const int groups = kTopkThreads / mpad;
  const int c = tid & (mpad - 1), g = tid / mpad;
  if (tid < kRankMax) rank[tid] = 0;
  __syncthreads();
  if (c < m) {
    const uint32_t u = cand_u[c], ps = cand_i[c];
    int larger = 0;
    for (int j = g; j < m; j += groups) {
      const uint32_t uj = cand_u[j], pj = cand_i[j];
      larger += (uj > u) || (uj == u && pj < ps);
    }
    if (larger) atomicAdd(&rank[c], larger);
  }
  __syncthreads();
  if (tid < m && rank[tid] == need - 1) { scratch[41] = (int)cand_u[tid]; scratch[42] = (int)cand_i[tid]; }
  __syncthreads();
  *prefix_out = (uint32_t)scratch[41];
  *pos_out = (uint32_t)scratch[42];
}

// Ordered output of the picks of [r_lo, r_hi) by one wavefront, 64 * kVec consecutive keys at a time with ballot prefix
// sums; `o` = number of picks before r_lo.  A key is picked iff  u > prefix || (u == prefix && position <= pos_thresh).
template <int kVec>
__device__ __forceinline__ void ordered_write(const float* x, const TopkSink& out, int r_lo, int r_hi, int lane, int o, int k,
                                              uint32_t prefix, uint32_t pos_thresh) {
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  constexpr int kWDepth = 4;
  for (int c0 = r_lo; c0 < r_hi; c0 += 64 * kVec * kWDepth) {
    float v[kWDepth][kVec];
#pragma unroll
    for (int j = 0; j < kWDepth; j++) {
      const int i = c0 + j * 64 * kVec + lane * kVec;
      if (kVec == 4 && i + 3 < r_hi) {
        const f32x4 q = *(const f32x4*)(x + i);
        v[j][0] = q[0]; v[j][1] = q[1]; v[j][2] = q[2]; v[j][3] = q[3];
      } else {
#pragma unroll
        for (int e = 0; e < kVec; e++) v[j][e] = i + e < r_hi ? x[i + e] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < kWDepth; j++) {
      const int i = c0 + j * 64 * kVec + lane * kVec;
      bool tk[kVec];
      int before = 0, total = 0;                              // picks of lower lanes / of the whole group of 64 * kVec keys
#pragma unroll
      for (int e = 0; e < kVec; e++) {
        const uint32_t u = ordered_bits(v[j][e]);
        tk[e] = i + e < r_hi && ((u > prefix) || (u == prefix && (uint32_t)(i + e) <= pos_thresh));
        const uint64_t m = __builtin_amdgcn_ballot_w64(tk[e]);
        before += __builtin_popcountll(m & below);
        total += __builtin_popcountll(m);
      }
      int at = o + before;
#pragma unroll
      for (int e = 0; e < kVec; e++)
        if (tk[e]) { if (at < k) out.put(at, i + e); at++; }
      o += total;
    }
  }
}

template <int kVec>
__global__ __launch_bounds__(kTopkThreads) void dsa_topk_kernel(const TopkParams p) {
  __shared__ int hist[kBins];
  __shared__ int scratch[64];
  __shared__ float fscratch[32];
  __shared__ uint32_t cand_u[kCandCap];
  __shared__ uint32_t cand_i[kCandCap];
  const int tid = threadIdx.x;
  const int lane = tid & 63, w = tid >> 6;
  const int b = blockIdx.x / p.max_q_len;
  const int ti = blockIdx.x - b * p.max_q_len;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  if (ti >= qlen) return;
  const int t = q0 + ti;
  int n = p.seq_lens[b] - qlen + ti + 1;                   // visible keys
  n = n < 0 ? 0 : n;
  const float* x = p.logits + (int64_t)t * p.l_st;
  const TopkSink out = topk_sink(p, b, t);
  const int k = p.k;
  if (p.counts && tid == 0) p.counts[t] = n < k ? n : k;

  if (n <= k) {                                            // everything is selected
    for (int i = tid; i < k; i += kTopkThreads) {
      if (i < n) out.put(i, i); else out.out[i] = -1;
    }
    return;
  }

  // ---- rough range of the finite logits from 4096 keys spread over the row (one round of loads) ----
  float lo = INFINITY, hi = -INFINITY;
  {
    const int step = n / 4096 > 0 ? n / 4096 : 1;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) { const int i = (tid + j * kTopkThreads) * step; v[j] = i < n ? x[i] : NAN; }
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (fabsf(v[j]) < INFINITY) { lo = fminf(lo, v[j]); hi = fmaxf(hi, v[j]); }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) { lo = fminf(lo, __shfl_xor(lo, o, 64)); hi = fmaxf(hi, __shfl_xor(hi, o, 64)); }
  if (lane == 0) { fscratch[w] = lo; fscratch[16 + w] = hi; }
  for (int i = tid; i < kBins; i += kTopkThreads) hist[i] = 0;
  if (tid == 0) scratch[40] = 0;                           // candidate counter
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; i++) { lo = fminf(lo, fscratch[i]); hi = fmaxf(hi, fscratch[16 + i]); }
  const float range = hi - lo;
  const float scale = (range > 0.f && range < INFINITY) ? (float)kBins * 0.99999f / range : 0.f;
  const float shift = scale != 0.f ? -lo * scale : 0.f;

  // ---- sweep 1: histogram over the linear bins; the bin that holds the k-th largest logit ----
  sweep<kVec>(x, 0, n, tid, kTopkThreads, [&](float v, int) { atomicAdd(&hist[linear_bin(v, scale, shift)], 1); });
  __syncthreads();
  int above;
  const int d = select_digit(hist, scratch, k, &above);
  int need = k - above;                                    // wanted among the keys of bin d (>= 1)
  const int in_bin = hist[d];
  __syncthreads();

  // Wavefront w owns the contiguous range [r_lo, r_hi) of the row for the ordered output.
  const int per = ((n + 15) / 16 + 255) / 256 * 256;
  const int r_lo = w * per;
  int r_hi = r_lo + per;
  r_hi = r_hi < n ? r_hi : n;

  // ---- sweep 2: the keys of bin d move to LDS, and every wavefront counts the sure picks (bins above d) of its range ----
  uint32_t prefix, pos_thresh;
  int cnt = 0;
  if (in_bin <= kCandCap) {
    sweep<kVec>(x, r_lo, r_hi, lane, 64, [&](float v, int i) {
      const int bn = linear_bin(v, scale, shift);
      cnt += bn > d;
      if (bn == d) {
        const int slot = atomicAdd(&scratch[40], 1);
        cand_u[slot] = ordered_bits(v);
        cand_i[slot] = (uint32_t)i;
      }
    });
    __syncthreads();
    if (in_bin <= kRankMax) {
      rank_threshold(cand_u, cand_i, in_bin, need, hist, scratch, &prefix, &pos_thresh);
    } else {
      radix_threshold<kTopkThreads>([&](auto&& f) { for (int j = tid; j < in_bin; j += kTopkThreads) f(cand_u[j], cand_i[j]); }, need, hist,
                      scratch, &prefix, &pos_thresh);
    }
    // candidates of my range that made it
    for (int j = lane; j < in_bin; j += 64) {
      const uint32_t u = cand_u[j], ps = cand_i[j];
      cnt += (int)ps >= r_lo && (int)ps < r_hi && ((u > prefix) || (u == prefix && ps <= pos_thresh));
    }
  } else {
    // degenerate rows (a large share of equal or nearly equal logits): the radix passes read the row itself
    radix_threshold<kTopkThreads>(
        [&](auto&& f) {
          sweep<kVec>(x, 0, n, tid, kTopkThreads, [&](float v, int i) {
            if (linear_bin(v, scale, shift) == d) f(ordered_bits(v), (uint32_t)i);
          });
        },
        need, hist, scratch, &prefix, &pos_thresh);
    sweep<kVec>(x, r_lo, r_hi, lane, 64, [&](float v, int i) {
      const uint32_t u = ordered_bits(v);
      cnt += (u > prefix) || (u == prefix && (uint32_t)i <= pos_thresh);
    });
  }
  // a key is selected iff  u > prefix || (u == prefix && position <= pos_thresh): keys of higher bins are larger than
  // every key of bin d, keys of lower bins smaller
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) cnt += __shfl_xor(cnt, o, 64);
  __syncthreads();
  if (lane == 0) scratch[w] = cnt;
  __syncthreads();
  int o = 0;
  for (int i = 0; i < w; i++) o += scratch[i];

  ordered_write<kVec>(x, out, r_lo, r_hi, lane, o, k, prefix, pos_thresh);
}

// ---- the same selection spread over several workgroups per token ------------------------------------------------
// One compute unit needs tens of microseconds for the ~12 vector instructions per key and sweep of a 64K-key row, so
// with few tokens in flight the row is cut into slices of kSliceKeys keys, one 1024-thread workgroup each (eight keys
// per thread, held in registers), and the three sweeps become three launches that meet in a workspace:
//   hist    slice histograms over the linear bins (every slice derives the same bins from the same sample of the row);
//   gather  every slice adds the histograms up, finds the boundary bin, counts its sure picks per wavefront and
//           appends its boundary-bin keys to the token's candidate list;
//   write   every slice finds the exact threshold among the candidates and writes its picks at their final places.
// A launch costs little more than its chain of dependent memory round trips (more than a microsecond each), so every
// kernel asks for all the global data it will need - its slice of the row included - before it looks at any of it.
constexpr int kMwWaves = kTopkThreads / 64;                // 16
constexpr int kSliceKeys = kTopkThreads * 8;               // 8192
constexpr int kMaxSlices = 16;                             // rows up to 131072 keys; longer ones take the one-workgroup kernel
constexpr int kMwCandLds = 4096;                           // candidates ranked / radix-selected in LDS; more: from memory

struct TopkMwParams {
  TopkParams t;
  int32_t slices;
  int32_t* hist_part;                                      // [tokens][slices][kBins]
  float* range;                                            // [tokens][2]: scale, shift
  int32_t* meta;                                           // [tokens][4]: candidate count, boundary bin, need, -
  int32_t* counts;                                         // [tokens][slices][kMwWaves] sure picks
  uint32_t* cand;                                          // [tokens][cand_cap][2]: ordered image, position
  int64_t cand_cap;
};

struct TopkRow { const float* x; int n, slot, b, t; bool live; };
__device__ __forceinline__ TopkRow topk_row(const TopkParams& p, int slot) {
  TopkRow r;
  const int b = slot / p.max_q_len;
  const int ti = slot - b * p.max_q_len;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  r.live = ti < qlen;
  const int t = q0 + ti;
  int n = p.seq_lens[b] - qlen + ti + 1;                   // visible keys
  r.n = n < 0 ? 0 : n;
  r.x = p.logits + (int64_t)t * p.l_st;
  r.b = b;
  r.t = t;
  r.slot = slot;
  return r;
}

// (slice, token slot) of a workgroup of the multi-workgroup kernels.  Workgroups go to the eight XCDs round-robin in launch
// order (x fastest); renumbered, every XCD takes a contiguous eighth of the tokens with all their slices, so what one kernel
// of the chain leaves for the next (slice histograms, candidates, counts, the logits themselves) is read through the XCD
// that wrote it.
struct SliceOf { int s, slot; };
__device__ __forceinline__ SliceOf slice_of_workgroup() {
  SliceOf r{(int)blockIdx.x, (int)blockIdx.y};
  const uint32_t total = gridDim.x * gridDim.y;
  if ((total & 7) == 0 && ((total >> 3) % gridDim.x) == 0) {
    const uint32_t lin = blockIdx.x + gridDim.x * blockIdx.y;
    const uint32_t nl = (lin & 7) * (total >> 3) + (lin >> 3);
    r.s = (int)(nl % gridDim.x);
    r.slot = (int)(nl / gridDim.x);
  }
  return r;
}

// This thread's eight keys of slice s: positions pos(j, e) = s*kSliceKeys + w*512 + j*256 + lane*4 + e (j < 2, e < 4), so
// that a wavefront holds 512 consecutive keys in (j, lane, e) order.  Keys at or past n read as 0 and are never used.
struct SliceKeys { float v[2][4]; int base; };
template <int kVec>
__device__ __forceinline__ SliceKeys load_slice(const float* x, int n, int s, int w, int lane) {
  SliceKeys k;
  k.base = s * kSliceKeys + w * 512 + lane * 4;
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int i = k.base + j * 256;
    if (kVec == 4 && i + 3 < n) {
      const f32x4 q = *(const f32x4*)(x + i);
      k.v[j][0] = q[0]; k.v[j][1] = q[1]; k.v[j][2] = q[2]; k.v[j][3] = q[3];
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) k.v[j][e] = i + e < n ? x[i + e] : 0.f;
    }
  }
  return k;
}

template <int kVec>
__global__ __launch_bounds__(kTopkThreads) void dsa_topk_hist_kernel(const TopkMwParams p) {
  __shared__ int hist[kBins];
  __shared__ float fscratch[2 * kMwWaves];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const SliceOf so = slice_of_workgroup();
  const int s = so.s;
  const TopkRow r = topk_row(p.t, so.slot);
  if (!r.live || r.n <= p.t.k || s * kSliceKeys >= r.n) return;
  const int n = r.n;
  // all loads first: four runs of 1024 consecutive keys spread over the whole row (the sample that fixes the bins, the
  // same in every slice), and this slice
  float sm[4];
#pragma unroll
  for (int j = 0; j < 4; j++) { const int i = (int)((int64_t)j * n / 4) + tid; sm[j] = i < n ? r.x[i] : NAN; }
  const SliceKeys ks = load_slice<kVec>(r.x, n, s, w, lane);
  float lo = INFINITY, hi = -INFINITY;
#pragma unroll
  for (int j = 0; j < 4; j++)
    if (fabsf(sm[j]) < INFINITY) { lo = fminf(lo, sm[j]); hi = fmaxf(hi, sm[j]); }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) { lo = fminf(lo, __shfl_xor(lo, o, 64)); hi = fmaxf(hi, __shfl_xor(hi, o, 64)); }
  if (lane == 0) { fscratch[w] = lo; fscratch[kMwWaves + w] = hi; }
  for (int i = tid; i < kBins; i += kTopkThreads) hist[i] = 0;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kMwWaves; i++) { lo = fminf(lo, fscratch[i]); hi = fmaxf(hi, fscratch[kMwWaves + i]); }
  const float range = hi - lo;
  const float scale = (range > 0.f && range < INFINITY) ? (float)kBins * 0.99999f / range : 0.f;
  const float shift = scale != 0.f ? -lo * scale : 0.f;
  if (s == 0 && tid == 0) {
    p.range[r.slot * 2] = scale;
    p.range[r.slot * 2 + 1] = shift;
    p.meta[r.slot * 4] = 0;                                // candidate counter for the gather launch
  }
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (ks.base + j * 256 + e < n) atomicAdd(&hist[linear_bin(ks.v[j][e], scale, shift)], 1);
  __syncthreads();
  int32_t* hp = p.hist_part + ((int64_t)r.slot * p.slices + s) * kBins;
  for (int i = tid; i < kBins; i += kTopkThreads) hp[i] = hist[i];
}

template <int kVec>
__global__ __launch_bounds__(kTopkThreads) void dsa_topk_gather_kernel(const TopkMwParams p) {
  __shared__ int hist[kBins];
  __shared__ int scratch[64];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const SliceOf so = slice_of_workgroup();
  const int s = so.s;
  const TopkRow r = topk_row(p.t, so.slot);
  if (!r.live || r.n <= p.t.k || s * kSliceKeys >= r.n) return;
  const int n = r.n;
  const int live_slices = (n + kSliceKeys - 1) / kSliceKeys;
  // all loads first: the slice histograms of the token (two bins per thread), the bin map, this slice
  const int32_t* hp = p.hist_part + (int64_t)r.slot * p.slices * kBins;
  int c0 = 0, c1 = 0;
  for (int j = 0; j < live_slices; j++) { c0 += hp[j * kBins + tid]; c1 += hp[j * kBins + kTopkThreads + tid]; }
  const float scale = p.range[r.slot * 2], shift = p.range[r.slot * 2 + 1];
  const SliceKeys ks = load_slice<kVec>(r.x, n, s, w, lane);
  hist[tid] = c0;
  hist[kTopkThreads + tid] = c1;
  __syncthreads();
  int above;
  const int d = select_digit(hist, scratch, p.t.k, &above);
  if (s == 0 && tid == 0) { p.meta[r.slot * 4 + 1] = d; p.meta[r.slot * 4 + 2] = p.t.k - above; }
  uint32_t* cand = p.cand + (int64_t)r.slot * p.cand_cap * 2;
  int cnt = 0;
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int i = ks.base + j * 256 + e;
      if (i < n) {
        const int bn = linear_bin(ks.v[j][e], scale, shift);
        cnt += bn > d;
        if (bn == d) {
          const int slot = atomicAdd(&p.meta[r.slot * 4], 1);
          cand[2 * (int64_t)slot] = ordered_bits(ks.v[j][e]);
          cand[2 * (int64_t)slot + 1] = (uint32_t)i;
        }
      }
    }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) cnt += __shfl_xor(cnt, o, 64);
  if (lane == 0) p.counts[((int64_t)r.slot * p.slices + s) * kMwWaves + w] = cnt;
}

template <int kVec>
__global__ __launch_bounds__(kTopkThreads) void dsa_topk_write_kernel(const TopkMwParams p) {
  __shared__ int hist[kBins];
  __shared__ int scratch[64];
  __shared__ uint32_t cand_u[kMwCandLds];
  __shared__ uint32_t cand_i[kMwCandLds];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const SliceOf so = slice_of_workgroup();
  const int s = so.s;
  const TopkRow r = topk_row(p.t, so.slot);
  if (!r.live) return;
  const int n = r.n, k = p.t.k;
  const TopkSink out = topk_sink(p.t, r.b, r.t);
  if (p.t.counts && s == 0 && tid == 0) p.t.counts[r.t] = n < k ? n : k;
  if (n <= k) {                                            // everything is selected
    if (s == 0)
      for (int i = tid; i < k; i += kTopkThreads) {
        if (i < n) out.put(i, i); else out.out[i] = -1;
      }
    return;
  }
  if (s * kSliceKeys >= n) return;
  // all loads first: the candidate list (its first kMwCandLds entries, whatever their number turns out to be), the
  // sure-pick counts of the wavefronts before mine, this slice
  const uint32_t* cand = p.cand + (int64_t)r.slot * p.cand_cap * 2;
  const int lim = p.cand_cap < kMwCandLds ? (int)p.cand_cap : kMwCandLds;
  uint32_t cu[kMwCandLds / kTopkThreads], ci[kMwCandLds / kTopkThreads];
#pragma unroll
  for (int q = 0; q < kMwCandLds / kTopkThreads; q++) {
    const int j = tid + q * kTopkThreads;
    const u32x2 pr = j < lim ? *(const u32x2*)(cand + 2 * (int64_t)j) : u32x2{0u, 0u};
    cu[q] = pr[0];
    ci[q] = pr[1];
  }
  const int32_t* cn = p.counts + (int64_t)r.slot * p.slices * kMwWaves;
  const int mine = s * kMwWaves + w;                       // < kMaxSlices * kMwWaves = 256: four per lane
  int part = 0;
#pragma unroll
  for (int q = 0; q < 4; q++) { const int j = lane + q * 64; part += j < mine ? cn[j] : 0; }
  const int m = p.meta[r.slot * 4], need = p.meta[r.slot * 4 + 2];
  const SliceKeys ks = load_slice<kVec>(r.x, n, s, w, lane);
#pragma unroll
  for (int q = 0; q < kMwCandLds / kTopkThreads; q++) { cand_u[tid + q * kTopkThreads] = cu[q]; cand_i[tid + q * kTopkThreads] = ci[q]; }
  __syncthreads();

  // ---- exact threshold among the m candidates (every slice of the token repeats this small piece of work) ----
  uint32_t prefix, pos_thresh;
  const bool in_lds = m <= kMwCandLds;
  if (m <= kRankMax) {
    rank_threshold(cand_u, cand_i, m, need, hist, scratch, &prefix, &pos_thresh);
  } else if (in_lds) {
    radix_threshold<kTopkThreads>([&](auto&& f) { for (int j = tid; j < m; j += kTopkThreads) f(cand_u[j], cand_i[j]); }, need,
                                  hist, scratch, &prefix, &pos_thresh);
  } else {
    // degenerate rows (a large share of equal or nearly equal logits)
    radix_threshold<kTopkThreads>(
        [&](auto&& f) { for (int j = tid; j < m; j += kTopkThreads) f(cand[2 * (int64_t)j], cand[2 * (int64_t)j + 1]); }, need,
        hist, scratch, &prefix, &pos_thresh);
  }

  // ---- where this wavefront's picks start: sure picks of everything before it + accepted candidates before it ----
  const int wlo = s * kSliceKeys + w * 512;
  for (int j = lane; j < m; j += 64) {
    const uint32_t u = in_lds ? cand_u[j] : cand[2 * (int64_t)j], ps = in_lds ? cand_i[j] : cand[2 * (int64_t)j + 1];
    part += (int)ps < wlo && ((u > prefix) || (u == prefix && ps <= pos_thresh));
  }
#pragma unroll
  for (int sh = 32; sh >= 1; sh >>= 1) part += __shfl_xor(part, sh, 64);
  int o = part;
  const uint64_t below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int i = ks.base + j * 256;
    bool tk[4];
    int before = 0, total = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const uint32_t u = ordered_bits(ks.v[j][e]);
      tk[e] = i + e < n && ((u > prefix) || (u == prefix && (uint32_t)(i + e) <= pos_thresh));
      const uint64_t mk = __builtin_amdgcn_ballot_w64(tk[e]);
      before += __builtin_popcountll(mk & below);
      total += __builtin_popcountll(mk);
    }
    int at = o + before;
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (tk[e]) { if (at < k) out.put(at, i + e); at++; }
    o += total;
  }
}

// Sparse-MLA row list: logical positions -> flat cache rows, dropping -1 / out-of-range entries, order kept.
struct RowsParams {
  const int32_t* indices; int64_t i_st;                    // [T, K]
  const int32_t* block_table; int64_t bt_stride; int32_t max_blocks;
  const int32_t* seq_lens; const int32_t* qsl;
  int32_t batch, max_q_len, k, page_size;
  int64_t num_pages;
  int32_t* rows; int64_t r_st;                             // [T, K] flat rows (page * page_size + offset)
  int32_t* counts;                                         // [T]
};

__global__ __launch_bounds__(256) void dsa_build_rows_kernel(const RowsParams p) {
  __shared__ int scratch[8];
  const int tid = threadIdx.x;
  const int b = blockIdx.x / p.max_q_len;
  const int ti = blockIdx.x - b * p.max_q_len;
  int q0, qlen;
  if (p.qsl) { q0 = p.qsl[b]; qlen = p.qsl[b + 1] - q0; } else { q0 = b * p.max_q_len; qlen = p.max_q_len; }
  if (ti >= qlen) return;
  const int t = q0 + ti;
  int n = p.seq_lens[b] - qlen + ti + 1;
  n = n < 0 ? 0 : n;
  const int32_t* idx = p.indices + (int64_t)t * p.i_st;
  int32_t* rows = p.rows + (int64_t)t * p.r_st;
  const int per = (p.k + 255) / 256;
  const int lo = tid * per;
  int hi = lo + per;
  hi = hi < p.k ? hi : p.k;
  int cnt = 0;
  for (int i = lo; i < hi; i++) { const int v = idx[i]; cnt += v >= 0 && v < n; }
  const int lane = tid & 63, w = tid >> 6;
  int s = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(s, o, 64);
    if (lane >= o) s += v;
  }
  if (lane == 63) scratch[w] = s;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < w; i++) base += scratch[i];
  int o = base + s - cnt;
  for (int i = lo; i < hi; i++) {
    const int v = idx[i];
    if (v >= 0 && v < n) {
      int pg = v / p.page_size;
      const int off = v - pg * p.page_size;
      pg = pg < p.max_blocks ? pg : p.max_blocks - 1;
      int64_t blk = p.block_table[(int64_t)b * p.bt_stride + pg];
      blk = blk < 0 ? 0 : (blk >= p.num_pages ? p.num_pages - 1 : blk);
      rows[o++] = (int32_t)(blk * p.page_size + off);
    }
  }
  if (tid == 255) p.counts[t] = base + s;                  // inclusive total of the last thread
}

}  // namespace mlahip
using namespace mlahip;

// slices per token in the multi-workgroup variant, or 0 when the one-workgroup kernel should run: rows too long for
// kMaxSlices slices, or so many tokens that one workgroup each already fills the chip
static int topk_slices(int64_t tokens, int64_t logits_stride) {
  const int64_t s = (logits_stride + kSliceKeys - 1) / kSliceKeys;
  if (s > kMaxSlices || s <= 1 || tokens >= 256) return 0;
  return (int)s;
}

extern "C" size_t dsa_topk_workspace_bytes(int32_t batch, int32_t max_q_len, int64_t logits_stride) {
  if (batch <= 0 || max_q_len <= 0 || logits_stride <= 0) return 0;
  const size_t tokens = (size_t)batch * max_q_len;
  return tokens * ((size_t)kMaxSlices * kBins * 4 + 8 + 16 + (size_t)kMaxSlices * kMwWaves * 4 + (size_t)logits_stride * 8);
}

static int topk_impl(const float* logits, int64_t logits_stride, const int32_t* seq_lens, const int32_t* query_start_loc,
                     int32_t batch, int32_t max_q_len, int32_t k, int32_t* out_indices, int64_t out_stride,
                     const int32_t* block_table, int64_t bt_stride, int32_t max_blocks, int32_t page_size, int64_t num_pages,
                     int32_t* rows, int64_t rows_stride, int32_t* counts, void* workspace, size_t workspace_bytes,
                     hipStream_t stream) {
  MLA_REQUIRE(logits && seq_lens && out_indices, MLA_ERR_NULL, "dsa_topk: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && k >= 1 && out_stride >= k, MLA_ERR_SHAPE,
              "dsa_topk: batch=%d max_q_len=%d k=%d out_stride=%lld", batch, max_q_len, k, (long long)out_stride);
  MLA_REQUIRE(logits_stride < (1ll << 22), MLA_ERR_SHAPE, "dsa_topk: at most 2^22 keys per row");
  if (batch == 0) return MLA_OK;
  TopkParams p{logits, logits_stride, seq_lens, query_start_loc, batch, max_q_len, k, out_indices, out_stride,
               block_table, bt_stride, max_blocks, page_size, num_pages, rows, rows_stride, counts};
  // rows that start on 16-byte boundaries are read four keys per load
  const bool vec = ((uintptr_t)logits % 16 == 0) && (logits_stride % 4 == 0);
  const int64_t tokens = (int64_t)batch * max_q_len;
  const int slices = topk_slices(tokens, logits_stride);
  if (!workspace || slices == 0) {
    if (vec) hipLaunchKernelGGL(dsa_topk_kernel<4>, dim3(batch * max_q_len), dim3(kTopkThreads), 0, stream, p);
    else hipLaunchKernelGGL(dsa_topk_kernel<1>, dim3(batch * max_q_len), dim3(kTopkThreads), 0, stream, p);
    return check_launch("dsa_topk_kernel");
  }
  const size_t need = dsa_topk_workspace_bytes(batch, max_q_len, logits_stride);
  MLA_REQUIRE(workspace_bytes >= need, MLA_ERR_WORKSPACE, "dsa_topk: workspace %zu bytes < required %zu", workspace_bytes, need);
  MLA_REQUIRE((uintptr_t)workspace % 16 == 0, MLA_ERR_SHAPE, "dsa_topk: workspace must be 16-byte aligned");
  TopkMwParams m;
  m.t = p;
  m.slices = slices;
  char* w = (char*)workspace;
  m.hist_part = (int32_t*)w; w += (size_t)tokens * kMaxSlices * kBins * 4;
  m.range = (float*)w; w += (size_t)tokens * 8;
  m.meta = (int32_t*)w; w += (size_t)tokens * 16;
  m.counts = (int32_t*)w; w += (size_t)tokens * kMaxSlices * kMwWaves * 4;
  m.cand = (uint32_t*)w;
  m.cand_cap = logits_stride;
  const dim3 grid(slices, (unsigned)tokens);
  if (vec) {
    hipLaunchKernelGGL(dsa_topk_hist_kernel<4>, grid, dim3(kTopkThreads), 0, stream, m);
    hipLaunchKernelGGL(dsa_topk_gather_kernel<4>, grid, dim3(kTopkThreads), 0, stream, m);
    hipLaunchKernelGGL(dsa_topk_write_kernel<4>, grid, dim3(kTopkThreads), 0, stream, m);
  } else {
    hipLaunchKernelGGL(dsa_topk_hist_kernel<1>, grid, dim3(kTopkThreads), 0, stream, m);
    hipLaunchKernelGGL(dsa_topk_gather_kernel<1>, grid, dim3(kTopkThreads), 0, stream, m);
    hipLaunchKernelGGL(dsa_topk_write_kernel<1>, grid, dim3(kTopkThreads), 0, stream, m);
  }
  return check_launch("dsa_topk (hist / gather / write)");
}

// workspace may be NULL: then one workgroup per token does all the work (no scratch memory at all).
extern "C" int dsa_topk(const float* logits, int64_t logits_stride, const int32_t* seq_lens, const int32_t* query_start_loc,
                        int32_t batch, int32_t max_q_len, int32_t k, int32_t* out_indices, int64_t out_stride,
                        void* workspace, size_t workspace_bytes, hipStream_t stream) {
  return topk_impl(logits, logits_stride, seq_lens, query_start_loc, batch, max_q_len, k, out_indices, out_stride, nullptr, 0,
                   1, 1, 1, nullptr, 0, nullptr, workspace, workspace_bytes, stream);
}

// dsa_topk and dsa_build_rows in one: besides the positions (the reference's index buffer) every pick is translated
// through the block table into its flat cache row, and counts[t] = number of picks of token t.
extern "C" int dsa_topk_rows(const float* logits, int64_t logits_stride, const int32_t* seq_lens,
                             const int32_t* query_start_loc, int32_t batch, int32_t max_q_len, int32_t k,
                             int32_t* out_indices, int64_t out_stride, const int32_t* block_table, int64_t bt_stride,
                             int32_t max_blocks, int32_t page_size, int64_t num_pages, int32_t* rows, int64_t rows_stride,
                             int32_t* counts, void* workspace, size_t workspace_bytes, hipStream_t stream) {
  MLA_REQUIRE(block_table && rows && counts, MLA_ERR_NULL, "dsa_topk_rows: null pointer argument");
  MLA_REQUIRE(page_size >= 1 && num_pages >= 1 && max_blocks >= 1 && rows_stride >= k && num_pages * page_size < (1ll << 31),
              MLA_ERR_SHAPE, "dsa_topk_rows: page_size=%d max_blocks=%d rows_stride=%lld", page_size, max_blocks,
              (long long)rows_stride);
  return topk_impl(logits, logits_stride, seq_lens, query_start_loc, batch, max_q_len, k, out_indices, out_stride, block_table,
                   bt_stride, max_blocks, page_size, num_pages, rows, rows_stride, counts, workspace, workspace_bytes, stream);
}

extern "C" int dsa_build_rows(const int32_t* indices, int64_t indices_stride, const int32_t* block_table, int64_t bt_stride,
                              int32_t max_blocks, const int32_t* seq_lens, const int32_t* query_start_loc, int32_t batch,
                              int32_t max_q_len, int32_t k, int32_t page_size, int64_t num_pages, int32_t* rows,
                              int64_t rows_stride, int32_t* counts, hipStream_t stream) {
  MLA_REQUIRE(indices && block_table && seq_lens && rows && counts, MLA_ERR_NULL, "dsa_build_rows: null pointer argument");
  MLA_REQUIRE(batch >= 0 && max_q_len >= 1 && k >= 1 && page_size >= 1 && num_pages >= 1 && max_blocks >= 1 &&
                  rows_stride >= k && indices_stride >= k && num_pages * page_size < (1ll << 31),
              MLA_ERR_SHAPE, "dsa_build_rows: batch=%d max_q_len=%d k=%d page_size=%d", batch, max_q_len, k, page_size);
  if (batch == 0) return MLA_OK;
  RowsParams p{indices, indices_stride, block_table, bt_stride, max_blocks, seq_lens, query_start_loc, batch, max_q_len,
               k, page_size, num_pages, rows, rows_stride, counts};
  hipLaunchKernelGGL(dsa_build_rows_kernel, dim3(batch * max_q_len), dim3(256), 0, stream, p);
  return check_launch("dsa_build_rows_kernel");
}
