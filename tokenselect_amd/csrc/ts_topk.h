// Shared declarations of the ragged top-k: workspace layout, kernel arguments and
// the key transform, used by ts_topk.hip, by the vote kernel (which can fill the
// first histogram while it writes the votes) and by the per-layer driver.
#pragma once

#include "ts_common.h"

namespace ts {

constexpr int kTopkBins = 2048;          // 11-bit digits
constexpr int kTopkSlice = 512;          // candidates per workgroup of the hist / mark grids
constexpr int kTopkFinalThreads = 1024;
// Per-request workspace, in 32-bit words:
//   [hist0: 2048][hist1: 2048][cand_count: 1, padded to 64]   <- zeroed before every selection
//   [bitmap: 1 bit per candidate, 64-bit words]
//   [candidate list: (key, position) pairs, up to one per candidate]
constexpr int kTopkHist0 = 0;
constexpr int kTopkHist1 = kTopkBins;
constexpr int kTopkCandCount = 2 * kTopkBins;
constexpr int kTopkCounterWords = 2 * kTopkBins + 64;

struct TopkArgs {
  const float* votes;
  int64_t vote_stride;
  const int32_t* seq_lens;
  const int32_t* table;
  int64_t table_stride;
  const int32_t* k_per_req;
  const int32_t* hit;
  int32_t* topk_cache;  // [B, top_k] or NULL
  int32_t* cache_len;   // [B] or NULL
  int n_init, n_local, top_k, page_size, page_shift, pool_kernel, max_seq_len;
  uint32_t pool_rows;
  int32_t* sel;
  int32_t* sel_pos;
  int64_t sel_stride;
  int32_t* sel_len;
  uint32_t* ws;
  size_t ws_stride;   // words per request
  int bitmap_words;   // 32-bit words of the bitmap region
  uint32_t cand_cap;  // entries of the candidate list
};

__device__ __host__ __forceinline__ uint32_t* topk_ws(uint32_t* ws, size_t stride, int b) {
  return ws + (size_t)b * stride;
}

// Monotone map fp32 -> uint32: larger float <=> larger key.
__device__ __forceinline__ uint32_t vote_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ uint32_t key_bin0(uint32_t key) { return key >> 21; }
__device__ __forceinline__ uint32_t key_bin1(uint32_t key) { return (key >> 10) & 2047u; }
__device__ __forceinline__ uint32_t key_bin2(uint32_t key) { return key & 1023u; }

size_t topk_ws_stride_words(int max_n);
TopkArgs make_topk_args(const ts_config* cfg, const ts_batch* bt, const float* votes,
                        int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                        int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                        uint32_t* workspace);
// zero: clear the counters first; hist: build the first histogram here (false when
// the vote kernel already did).
int launch_topk(const TopkArgs& a, int batch, int max_n, bool zero, bool hist, hipStream_t stream);

}  // namespace ts
