// Shared declarations of the ragged top-k: workspace layout, kernel arguments, the
// key transform and the histogram search, used by ts_topk.hip, by the fused
// selection kernel and by the per-layer driver.
#pragma once

#include "ts_common.h"

namespace ts {

constexpr int kTopkBins = 2048;          // 11-bit digits
constexpr int kTopkSlice = 512;          // least candidates per workgroup of the hist / mark grids
constexpr int kTopkFinalThreads = 1024;
constexpr int kTopkPartWords = 512;      // 32-bit bitmap words per workgroup of the final grid
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
  int slice;          // candidates per workgroup of the hist / mark grids (set by launch_topk)
  // Words the last kernel clears for whoever runs next on the stream (the
  // attention's tickets): clear_per_req words per request, or NULL.
  uint32_t* clear;
  int clear_per_req;
  // A word an earlier kernel of the stream leaves non-zero when the votes are not
  // valid (a wait of the fused scoring gave up): sel_len then reports -1.  Or NULL.
  const uint32_t* fault;
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

// Block-wide search of a descending histogram: finds the bin t such that
// count(bins > t) < need <= count(bins >= t).  `hist` has NB entries (global or
// LDS) per copy, NB a multiple of blockDim.x; COPIES consecutive copies are added
// up.  Returns t and count(bins > t) to every thread.  `scratch` is LDS of
// blockDim.x/64 + 2 words.  VECTOR: the number of threads of the workgroup, given at
// compile time when `hist` is 16-byte aligned global memory (vector loads).
// The search comes in two halves, so that a caller can request the bins of several
// histograms (and whatever else it needs from memory) before it searches the first: the
// searches end in barriers that later loads would wait behind.
template <int NB, int COPIES = 1, int VECTOR = 0>
__device__ __forceinline__ void load_threshold_bins(const uint32_t* hist, uint32_t (&local)[8]) {
  const int tid = threadIdx.x, nthreads = VECTOR ? VECTOR : (int)blockDim.x;
  const int per = NB / nthreads;  // bins per thread, thread 0 owns the highest bins
  const int hi_bin = NB - 1 - tid * per;
#pragma unroll
  for (int i = 0; i < 8; ++i) local[i] = 0;
  if (VECTOR && (per == 8 || per == 4 || per == 2)) {
    // The thread's bins as one or two aligned vector loads (ascending addresses, taken in
    // descending order below): eight separate loads per thread, each wave instruction
    // strided over 2 KB, made this search 5 us of the top-k mark kernel.
#pragma unroll
    for (int c = 0; c < COPIES; ++c) {
      const uint32_t* base = hist + c * NB + (NB - (tid + 1) * per);
      uint32_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (per == 8) {
        const uint4 a = ((const uint4*)base)[0], b = ((const uint4*)base)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
      } else if (per == 4) {
        const uint4 a = ((const uint4*)base)[0];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
      } else {
        const uint2 a = ((const uint2*)base)[0];
        v[0] = a.x; v[1] = a.y;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (i < per) local[i] += v[per - 1 - i];
    }
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < per) {
#pragma unroll
        for (int c = 0; c < COPIES; ++c) local[i] += hist[c * NB + hi_bin - i];
      }
  }
}

template <int NB, int VECTOR = 0>
__device__ __forceinline__ void search_threshold_bins(const uint32_t (&local)[8], uint32_t need,
                                                      uint32_t* scratch, uint32_t& t_out,
                                                      uint32_t& above_out) {
  const int tid = threadIdx.x, nthreads = VECTOR ? VECTOR : (int)blockDim.x;
  const int per = NB / nthreads;
  const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
  const int hi_bin = NB - 1 - tid * per;
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (i < per) mine += local[i];
  // exclusive prefix of `mine` over threads (descending bins)
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) scratch[wave] = incl;
  if (tid == 0) {
    scratch[nwaves] = 0;
    scratch[nwaves + 1] = 0;
  }
  __syncthreads();
  uint32_t wave_base = 0;
  for (int w = 0; w < wave; ++w) wave_base += scratch[w];
  const uint32_t before = wave_base + incl - mine;  // count in bins above this thread's range
  if (before < need && need <= before + mine) {      // the crossing lies in this thread's bins
    uint32_t run = before;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < per) {
        if (run < need && need <= run + local[i]) {
          scratch[nwaves] = (uint32_t)(hi_bin - i);
          scratch[nwaves + 1] = run;
        }
        run += local[i];
      }
  }
  __syncthreads();
  t_out = scratch[nwaves];
  above_out = scratch[nwaves + 1];
  __syncthreads();
}

template <int NB, int COPIES = 1, int VECTOR = 0>
__device__ __forceinline__ void find_threshold_bin(const uint32_t* hist, uint32_t need,
                                                   uint32_t* scratch, uint32_t& t_out,
                                                   uint32_t& above_out) {
  uint32_t local[8];
  load_threshold_bins<NB, COPIES, VECTOR>(hist, local);
  search_threshold_bins<NB, VECTOR>(local, need, scratch, t_out, above_out);
}

size_t topk_ws_stride_words(int max_n);
TopkArgs make_topk_args(const ts_config* cfg, const ts_batch* bt, const float* votes,
                        int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                        int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                        uint32_t* workspace);
// counters_zeroed: an earlier kernel of the stream cleared the per-request counters
// (topk_zero_region() says where they are); hist0_filled: the vote kernel was given
// the workspace and has counted the first-level histogram already.
int launch_topk(const TopkArgs& a, int batch, int max_n, hipStream_t stream,
                bool counters_zeroed = false, bool hist0_filled = false);
ZeroRegion topk_zero_region(const TopkArgs& a, int batch);

// Max-pool of the votes (ts_vote.hip, tr.py:366-369): pooled[t] over votes[t - pad, t - pad + kernel).
int launch_pool(const ts_config* cfg, const ts_batch* bt, const float* votes, int64_t vote_stride,
                float* pooled, int64_t pooled_stride, const int32_t* skip, hipStream_t stream);

// Soft vote (ts_vote.hip); with hist_ws (the top-k workspace, counters zeroed) the vote
// kernel also fills the first-level histogram of the selection, unless max-pooling
// comes between the votes and the selection.
int launch_vote(const ts_config* cfg, const ts_batch* bt, const float* scores, int64_t score_stride,
                const float* partials, const int32_t* skip, float* stats, float* votes,
                float* pooled, int64_t vote_stride, uint32_t* hist_ws, size_t hist_ws_stride,
                hipStream_t stream);

}  // namespace ts
