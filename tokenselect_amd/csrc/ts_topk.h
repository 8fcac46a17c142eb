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
//   [hist0: 8 x 2048][hist1: 2048][cand_count: 1, padded to 64]   <- zeroed before every selection
//   [bitmap: 1 bit per candidate, 64-bit words]
//   [candidate list: (key, position) pairs, up to one per candidate]
// The first histogram is kept in kTopkHistCopies copies that its readers add up:
// the votes of a request fall into a few dozen adjacent bins, i.e. one or two cache
// lines, and hundreds of workgroups adding to the same line serialise in memory.
constexpr int kTopkHistCopies = 8;
constexpr int kTopkHist0 = 0;
constexpr int kTopkHist1 = kTopkHistCopies * kTopkBins;
constexpr int kTopkCandCount = kTopkHist1 + kTopkBins;
constexpr int kTopkCounterWords = kTopkCandCount + 64;
// Behind the per-request pieces lies the rendezvous area of the fused score + vote
// kernel, cleared together with the counters: kSyncSlots + 1 slots of two live
// words, kSyncSlotWords apart so that the slots fall into different memory
// channels.  Slot 0: [arrival counter, fault flag]; slot 1 + r: [round reached]
// replica r, polled by the workgroups with index % kSyncSlots == r.
constexpr int kSyncSlots = 64;
constexpr int kSyncSlotWords = 1024;
constexpr size_t kSyncWords = (size_t)(kSyncSlots + 1) * kSyncSlotWords;

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
  // Words the last kernel clears for whoever runs next on the stream (the
  // attention's tickets): clear_per_req words per request, or NULL.
  uint32_t* clear;
  int clear_per_req;
};

__device__ __host__ __forceinline__ uint32_t* topk_ws(uint32_t* ws, size_t stride, int b) {
  return ws + (size_t)b * stride;
}

// Monotone map fp32 -> uint32: larger float <=> larger key.
__device__ __forceinline__ uint32_t vote_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// The copy of the first histogram that workgroup `block` of a request adds to.
__device__ __forceinline__ uint32_t* hist0_copy(uint32_t* request_ws, unsigned block) {
  return request_ws + kTopkHist0 + (block % kTopkHistCopies) * kTopkBins;
}
__device__ __forceinline__ uint32_t key_bin0(uint32_t key) { return key >> 21; }
__device__ __forceinline__ uint32_t key_bin1(uint32_t key) { return (key >> 10) & 2047u; }
__device__ __forceinline__ uint32_t key_bin2(uint32_t key) { return key & 1023u; }

size_t topk_ws_stride_words(int max_n);
// First word of the rendezvous area inside a workspace of `batch` requests.
inline uint32_t* topk_sync_area(void* workspace, int batch, int max_n) {
  return (uint32_t*)workspace + align_up(topk_ws_stride_words(max_n) * (size_t)batch, 64);
}
TopkArgs make_topk_args(const ts_config* cfg, const ts_batch* bt, const float* votes,
                        int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                        int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                        uint32_t* workspace);
// zero: clear the counters first; hist: build the first histogram here (false when
// the vote kernel already did).
int launch_topk(const TopkArgs& a, int batch, int max_n, bool zero, bool hist, hipStream_t stream);

}  // namespace ts
