// Ragged top-k, ascending sort and index assembly (tr.py:371-373, 433-449).
//
// Exact radix select on order-preserving 32-bit keys of the fp32 votes, split
// 11 + 11 + 10 bits, spread over many workgroups:
//
//   hist   (grid over candidates)  histogram of the top 11 key bits per request
//   mark   (grid over candidates)  finds the threshold bin t0; every candidate in
//                                  a higher bin is selected for sure and gets its
//                                  bit in a position bitmap (one plain 64-bit
//                                  store per wavefront); candidates inside bin t0
//                                  are appended to a short list and histogrammed
//                                  on their next 11 bits
//   final  (a few workgroups per request, one per slice of the bitmap) resolves
//                                  the remaining 21 bits on the short list (ties
//                                  at the k-th key: lowest position first), sets
//                                  their bits, then walks its slice of the bitmap
//                                  with a popcount prefix scan and emits the
//                                  selected positions in ascending order, together
//                                  with the sink and local-window segments and
//                                  the logical -> physical translation.
//
// The output is sorted without a sort and bit-stable across runs (no result
// depends on the order in which atomics land).
#include <stdlib.h>

#include "ts_topk.h"

namespace ts {

__device__ __forceinline__ int pooled_count(int n, int pool_kernel) {
  return (pool_kernel > 0 && (pool_kernel & 1) == 0) ? n - 1 : n;  // even kernel: one fewer
}

__global__ __launch_bounds__(256) void topk_zero_kernel(uint32_t* __restrict__ ws,
                                                        size_t stride_words) {
  uint32_t* p = ws + (size_t)blockIdx.x * stride_words;
  for (int i = threadIdx.x; i < kTopkCounterWords; i += 256) p[i] = 0u;
}

__global__ __launch_bounds__(256) void topk_hist_kernel(TopkArgs a) {
  const int b = blockIdx.y;
  if (a.hit && a.hit[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int n = pooled_count(geo.n, a.pool_kernel);
  const int lo = blockIdx.x * a.slice;
  if (lo >= n) return;
  __shared__ uint32_t lh[kTopkBins];
  for (int i = threadIdx.x; i < kTopkBins; i += 256) lh[i] = 0u;
  __syncthreads();
  const float* votes = a.votes + (int64_t)b * a.vote_stride;
  for (int i = lo + threadIdx.x; i < min(lo + a.slice, n); i += 256)
    atomicAdd(&lh[key_bin0(vote_key(votes[i]))], 1u);
  __syncthreads();
  uint32_t* hist0 = topk_ws(a.ws, a.ws_stride, b) + kTopkHist0;
  for (int i = threadIdx.x; i < kTopkBins; i += 256)
    if (lh[i]) atomicAdd(&hist0[i], lh[i]);
}

__global__ __launch_bounds__(256) void topk_mark_kernel(TopkArgs a) {
  const int b = blockIdx.y;
  if (a.hit && a.hit[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int n = pooled_count(geo.n, a.pool_kernel);
  const int lo = blockIdx.x * a.slice;
  if (lo >= n) return;

  __shared__ uint32_t scratch[8];
  __shared__ uint32_t lh[kTopkBins];
  uint32_t* ws = topk_ws(a.ws, a.ws_stride, b);
  // The votes of the slice are requested together with the histogram: they arrive while
  // the threshold bin is searched for.
  const float* votes = a.votes + (int64_t)b * a.vote_stride;
  const int lane = threadIdx.x & 63;
  const int first = lo + (threadIdx.x & ~63);
  const int end = min(lo + a.slice, n);
  constexpr int kAhead = 4096 / 256;  // passes of the largest slice
  uint32_t bins0[8];
  load_threshold_bins<kTopkBins, 1, 256>(ws + kTopkHist0, bins0);
  float ahead[kAhead];
#pragma unroll
  for (int it = 0; it < kAhead; ++it) {
    const int i = first + 256 * it + lane;
    ahead[it] = (first + 256 * it < end && i < n) ? votes[i] : 0.f;
  }
  uint32_t t0, above0;
  search_threshold_bins<kTopkBins, 256>(bins0, (uint32_t)geo.k, scratch, t0, above0);
  for (int i = threadIdx.x; i < kTopkBins; i += 256) lh[i] = 0u;
  __syncthreads();

  uint64_t* bitmap = (uint64_t*)(ws + kTopkCounterWords);
  uint2* cand = (uint2*)(ws + kTopkCounterWords + a.bitmap_words);
  // Whole 64-position groups per wave iteration so that a bitmap word has one writer.
#pragma unroll
  for (int it = 0; it < kAhead; ++it) {
    const int base = first + 256 * it;
    if (base >= end) break;
    const int i = base + lane;
    uint32_t key = 0;
    bool gt = false, eq = false;
    if (i < n) {
      key = vote_key(ahead[it]);
      const uint32_t bin = key_bin0(key);
      gt = bin > t0;
      eq = bin == t0;
    }
    const uint64_t gt_mask = __ballot(gt), eq_mask = __ballot(eq);
    if (lane == 0) bitmap[base >> 6] = gt_mask;
    if (eq_mask) {
      uint32_t slot = 0;
      if (lane == 0) slot = atomicAdd(&ws[kTopkCandCount], (uint32_t)__popcll(eq_mask));
      slot = __shfl(slot, 0);
      if (eq) {
        const uint32_t at = slot + __popcll(eq_mask & ((1ull << lane) - 1ull));
        if (at < a.cand_cap) cand[at] = make_uint2(key, (uint32_t)i);  // cap: counters not cleared
        atomicAdd(&lh[key_bin1(key)], 1u);
      }
    }
  }
  __syncthreads();
  uint32_t* hist1 = ws + kTopkHist1;
  for (int i = threadIdx.x; i < kTopkBins; i += 256)
    if (lh[i]) atomicAdd(&hist1[i], lh[i]);
}

__global__ __launch_bounds__(kTopkFinalThreads) void topk_final_kernel(TopkArgs a) {
  const int b = blockIdx.y;
  const int part = blockIdx.x, parts = gridDim.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;
  int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
  int32_t* sel_pos = a.sel_pos + (int64_t)b * a.sel_stride;
  const int L = geo.seq_len;
  // This thread's share of a loop that the request's workgroups walk together.
  const int first = part * kTopkFinalThreads + tid, step = parts * kTopkFinalThreads;
  if (a.clear && part == 0)
    for (int i = tid; i < a.clear_per_req; i += kTopkFinalThreads)
      a.clear[(size_t)b * a.clear_per_req + i] = 0u;

  auto emit = [&](int out_idx, int pos) {
    sel_pos[out_idx] = pos;
    sel[out_idx] = (int32_t)lookup_slot(tab, pos, a.page_size, a.page_shift, a.pool_rows);
  };

  if (geo.dense) {  // tr.py:377-378, 741-744: attend over every token
    for (int i = first; i < L; i += step) emit(i, i);
    if (part == 0 && tid == 0) a.sel_len[b] = L;
    return;
  }
  const bool is_hit = a.hit && a.hit[b];
  const int k = is_hit ? min(a.cache_len[b], a.top_k) : geo.k;
  if (part == 0 && tid == 0)
    a.sel_len[b] = (a.fault && !is_hit && *a.fault) ? -1 : a.n_init + k + a.n_local;
  for (int i = first; i < a.n_init; i += step) emit(i, i);
  for (int i = first; i < a.n_local; i += step) emit(a.n_init + k + i, L - a.n_local + i);
  if (is_hit) {  // tr.py:419: reuse the cached positions
    const int32_t* cached = a.topk_cache + (int64_t)b * a.top_k;
    for (int i = first; i < k; i += step) emit(a.n_init + i, cached[i]);
    return;
  }

  // The workgroups of a request split the position bitmap into consecutive slices
  // of whole 32-bit words.  Each resolves the k-th key on its own (the histograms
  // and the short list are small), sets the bits of the listed candidates that
  // fall into its slice in an LDS copy, counts the selected positions before the
  // slice, and emits its slice; no workgroup waits for another.
  const int n = pooled_count(geo.n, a.pool_kernel);
  const int words = (n + 31) >> 5;
  const int per_part = (words + parts - 1) / parts;  // <= kTopkPartWords by the launch grid
  const int w_lo = min(part * per_part, words), w_hi = min(w_lo + per_part, words);
  if (w_lo >= w_hi) return;
  uint32_t* ws = topk_ws(a.ws, a.ws_stride, b);
  const uint32_t* bitmap32 = ws + kTopkCounterWords;
  const uint2* cand = (const uint2*)(ws + kTopkCounterWords + a.bitmap_words);
  const int ncand = (int)min(ws[kTopkCandCount], (uint32_t)n);

  __shared__ uint32_t scratch[kTopkFinalThreads / 64 + 2];
  __shared__ uint32_t lh[1024];
  __shared__ uint32_t lbits[kTopkPartWords];
  // Both histograms are requested before anything else is waited for: the searches
  // below end in barriers that their loads would otherwise queue behind.
  uint32_t bins0[8], bins1[8];
  load_threshold_bins<kTopkBins, 1, kTopkFinalThreads>(ws + kTopkHist0, bins0);
  load_threshold_bins<kTopkBins, 1, kTopkFinalThreads>(ws + kTopkHist1, bins1);
  // ... and this thread's first entry of the short list (the list rarely has more entries
  // than the workgroup has threads; one past its end is never used).
  const uint2 cand_first = (uint32_t)tid < a.cand_cap ? cand[tid] : make_uint2(0u, 0u);
  auto cand_at = [&](int i) { return i == tid ? cand_first : cand[i]; };
  uint32_t before = 0;  // selected positions before the slice, this thread's share
  for (int w = tid; w < w_lo; w += kTopkFinalThreads) before += __popc(bitmap32[w]);
  for (int w = w_lo + tid; w < w_hi; w += kTopkFinalThreads) {
    uint32_t bits = bitmap32[w];
    const int rem = n - (w << 5);
    if (rem < 32) bits &= (1u << rem) - 1u;  // positions past n hold stale bits
    lbits[w - w_lo] = bits;
  }
  auto mark = [&](uint32_t pos) {
    const int w = (int)(pos >> 5);
    if (w < w_lo)
      ++before;
    else if (w < w_hi)
      atomicOr(&lbits[w - w_lo], 1u << (pos & 31u));
  };

  uint32_t t0, above0, t1, above1, t2, above2;
  search_threshold_bins<kTopkBins, kTopkFinalThreads>(bins0, (uint32_t)k, scratch, t0, above0);
  const uint32_t need1 = (uint32_t)k - above0;  // still to take inside bin t0
  search_threshold_bins<kTopkBins, kTopkFinalThreads>(bins1, need1, scratch, t1, above1);
  const uint32_t need2 = need1 - above1;  // still to take inside (t0, t1)

  for (int i = tid; i < 1024; i += kTopkFinalThreads) lh[i] = 0u;
  __syncthreads();
  for (int i = tid; i < ncand; i += kTopkFinalThreads) {
    const uint2 c = cand_at(i);
    const uint32_t b1 = key_bin1(c.x);
    if (b1 > t1)
      mark(c.y);
    else if (b1 == t1)
      atomicAdd(&lh[key_bin2(c.x)], 1u);
  }
  __syncthreads();
  find_threshold_bin<1024>(lh, need2, scratch, t2, above2);
  const uint32_t need_eq = need2 - above2;  // ties at the k-th key still to take
  const uint32_t count_eq = lh[t2];
  __syncthreads();

  if (count_eq == need_eq) {  // the usual case: every tie is selected
    for (int i = tid; i < ncand; i += kTopkFinalThreads) {
      const uint2 c = cand_at(i);
      if (key_bin1(c.x) == t1 && key_bin2(c.x) >= t2) mark(c.y);
    }
  } else {
    // More ties than places: keep the need_eq lowest positions.  Positions are
    // unique, so a two-digit radix select on the position finds the largest one kept.
    uint32_t p_hi, p_lo, skip_hi, skip_lo;
    for (int i = tid; i < 1024; i += kTopkFinalThreads) lh[i] = 0u;
    __syncthreads();
    auto is_tie = [&](const uint2& c) { return key_bin1(c.x) == t1 && key_bin2(c.x) == t2; };
    for (int i = tid; i < ncand; i += kTopkFinalThreads) {
      const uint2 c = cand[i];
      if (is_tie(c)) atomicAdd(&lh[1023u - (c.y >> 10)], 1u);  // descending bin = ascending position
    }
    __syncthreads();
    find_threshold_bin<1024>(lh, need_eq, scratch, p_hi, skip_hi);
    const uint32_t pos_hi = 1023u - p_hi;
    for (int i = tid; i < 1024; i += kTopkFinalThreads) lh[i] = 0u;
    __syncthreads();
    for (int i = tid; i < ncand; i += kTopkFinalThreads) {
      const uint2 c = cand[i];
      if (is_tie(c) && (c.y >> 10) == pos_hi) atomicAdd(&lh[1023u - (c.y & 1023u)], 1u);
    }
    __syncthreads();
    find_threshold_bin<1024>(lh, need_eq - skip_hi, scratch, p_lo, skip_lo);
    const uint32_t last_pos = (pos_hi << 10) | (1023u - p_lo);
    for (int i = tid; i < ncand; i += kTopkFinalThreads) {
      const uint2 c = cand[i];
      if (key_bin1(c.x) == t1 && (key_bin2(c.x) > t2 || (key_bin2(c.x) == t2 && c.y <= last_pos)))
        mark(c.y);
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) before += __shfl_xor(before, off);
  if (lane == 0) scratch[wave] = before;
  __syncthreads();
  uint32_t running = 0;  // selected positions before the words handled so far
#pragma unroll
  for (int x = 0; x < kTopkFinalThreads / 64; ++x) running += scratch[x];
  __syncthreads();

  // Ordered emission: popcount prefix scan over the slice, one word per thread per round.
  int32_t* cache_out = a.topk_cache ? a.topk_cache + (int64_t)b * a.top_k : nullptr;
  for (int base = w_lo; base < w_hi; base += kTopkFinalThreads) {
    const int w = base + tid;
    uint32_t bits = w < w_hi ? lbits[w - w_lo] : 0u;
    const uint32_t cnt = __popc(bits);
    uint32_t incl = cnt;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const uint32_t up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    if (lane == 63) scratch[wave] = incl;
    __syncthreads();
    uint32_t wave_base = 0, total = 0;
#pragma unroll
    for (int x = 0; x < kTopkFinalThreads / 64; ++x) {
      const uint32_t s = scratch[x];
      if (x < wave) wave_base += s;
      total += s;
    }
    uint32_t out = running + wave_base + incl - cnt;
    while (bits) {
      const int bit = __ffs(bits) - 1;
      bits &= bits - 1u;
      if (out < (uint32_t)k) {
        const int pos = a.n_init + (w << 5) + bit;
        emit(a.n_init + (int)out, pos);
        if (cache_out) cache_out[out] = pos;
      }
      ++out;
    }
    running += total;
    __syncthreads();
  }
  if (part == 0 && tid == 0 && a.cache_len) a.cache_len[b] = k;
}

static size_t bitmap_words_for(int max_n) {
  return align_up((size_t)ceil_div(max_n > 0 ? max_n : 1, 64) * 2, 64);
}

size_t topk_ws_stride_words(int max_n) {
  return align_up(kTopkCounterWords + bitmap_words_for(max_n) + (size_t)(max_n > 0 ? max_n : 1) * 2,
                  64);
}

TopkArgs make_topk_args(const ts_config* cfg, const ts_batch* bt, const float* votes,
                        int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                        int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                        uint32_t* workspace) {
  TopkArgs a;
  a.votes = votes;
  a.vote_stride = vote_stride;
  a.seq_lens = bt->seq_lens;
  a.table = bt->table;
  a.table_stride = bt->table_stride;
  a.k_per_req = bt->k_per_req;
  a.hit = hit;
  a.topk_cache = cache ? cache->topk_cache : nullptr;
  a.cache_len = cache ? cache->cache_len : nullptr;
  a.n_init = cfg->n_init;
  a.n_local = cfg->n_local;
  a.top_k = cfg->top_k;
  a.max_seq_len = bt->max_seq_len;
  a.page_size = cfg->page_size;
  a.page_shift = page_shift_of(cfg->page_size);
  a.pool_kernel = cfg->pool_kernel;
  a.pool_rows = 0x7fffffffu;  // slots are not dereferenced here
  a.sel = sel;
  a.sel_pos = sel_pos;
  a.sel_stride = sel_stride;
  a.sel_len = sel_len;
  a.ws = workspace;
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  a.bitmap_words = (int)bitmap_words_for(max_n);
  a.cand_cap = (uint32_t)(max_n > 0 ? max_n : 1);
  a.ws_stride = topk_ws_stride_words(max_n);
  a.clear = nullptr;
  a.clear_per_req = 0;
  a.fault = nullptr;
  a.slice = kTopkSlice;
  return a;
}

ZeroRegion topk_zero_region(const TopkArgs& a, int batch) {
  ZeroRegion r;
  r.base = a.ws;
  r.stride = (int64_t)a.ws_stride;
  r.words = kTopkCounterWords;
  r.count = batch;
  return r;
}

// Candidates per workgroup of the hist / mark grids: every workgroup first searches
// the first-level histogram on its own, so a large batch gets larger slices (about a
// thousand workgroups in all), in multiples of the 256 candidates of a pass.
static int topk_slice(int batch, int max_n) {
  const int64_t per = ceil_div(ceil_div((int64_t)batch * max_n, 1024), 256) * 256;
  return (int)(per < kTopkSlice ? kTopkSlice : (per > 4096 ? 4096 : per));
}

int launch_topk(const TopkArgs& args, int batch, int max_n, hipStream_t stream, bool counters_zeroed,
                bool hist0_filled) {
  TopkArgs a = args;
  a.slice = topk_slice(batch, max_n);
  if (max_n > 0) {
    const dim3 grid((unsigned)ceil_div(max_n, a.slice), (unsigned)batch);
    if (!counters_zeroed) {
      hipLaunchKernelGGL(topk_zero_kernel, dim3((unsigned)batch), dim3(256), 0, stream, a.ws,
                         a.ws_stride);
      TS_TRY(check_launch("topk_zero_kernel"));
    }
    if (!hist0_filled) {
      hipLaunchKernelGGL(topk_hist_kernel, grid, dim3(256), 0, stream, a);
      TS_TRY(check_launch("topk_hist_kernel"));
    }
    hipLaunchKernelGGL(topk_mark_kernel, grid, dim3(256), 0, stream, a);
    TS_TRY(check_launch("topk_mark_kernel"));
  }
  const int parts = max_n > 0 ? ceil_div(ceil_div(max_n, 32), kTopkPartWords) : 1;
  hipLaunchKernelGGL(topk_final_kernel, dim3((unsigned)parts, (unsigned)batch),
                     dim3(kTopkFinalThreads), 0, stream, a);
  return check_launch("topk_final_kernel");
}

}  // namespace ts

using namespace ts;

extern "C" {

size_t ts_topk_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  const int max_n = max_seq_len - cfg->n_init - cfg->n_local;
  return align_up(topk_ws_stride_words(max_n) * 4 * (size_t)batch, 256);
}

int ts_topk_ragged(const ts_config* cfg, const ts_batch* bt, const float* votes,
                   int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                   int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                   void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(votes && sel && sel_pos && sel_len, TS_EINVAL, "ts_topk_ragged: NULL tensor argument");
  const int max_sel = cfg->n_init + cfg->top_k + cfg->n_local;
  TS_REQUIRE(sel_stride >= max_sel, TS_EWORKSPACE, "sel_stride %lld < n_init+top_k+n_local = %d",
             (long long)sel_stride, max_sel);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  // Ties at the k-th vote are cut by position, resolved as two 10-bit digits.
  TS_REQUIRE(max_n <= (1 << 20), TS_ESHAPE,
             "ts_topk_ragged: at most 2^20 candidates per request (max_seq_len %d)", bt->max_seq_len);
  TS_REQUIRE(hit == nullptr || cache != nullptr, TS_EINVAL,
             "ts_topk_ragged: hit flags need the selection cache");
  if (cache)
    TS_REQUIRE(cache->topk_cache && cache->cache_len, TS_EINVAL,
               "ts_topk_ragged: selection cache has a NULL array");
  const size_t need = ts_topk_workspace_bytes(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= need, TS_EWORKSPACE,
             "ts_topk_ragged: workspace %zu bytes < required %zu", workspace_bytes, need);
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  const TopkArgs a = make_topk_args(cfg, bt, votes, vote_stride, hit, cache, sel, sel_pos,
                                    sel_stride, sel_len, (uint32_t*)workspace);
  return launch_topk(a, bt->batch, max_n, (hipStream_t)stream);
}

}  // extern "C"
