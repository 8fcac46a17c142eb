// Ragged top-k, ascending sort and index assembly (tr.py:371-373, 433-449).
//
// One workgroup per request runs an exact radix select over order-preserving
// 32-bit keys of the fp32 votes (four 8-bit passes with an LDS histogram),
// which yields the k-th largest key T and how many elements equal to T are
// needed.  A single ordered compaction pass then emits, in ascending position,
// every element above T plus the lowest-positioned ties at T: the output is
// sorted without a sort and is bit-stable across runs.  The same kernel writes
// the sink and local-window segments and translates logical positions to
// physical slots through the table.
#include "ts_common.h"

namespace ts {

constexpr int kTopkThreads = 1024;
constexpr int kTopkWaves = kTopkThreads / 64;

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
};

// Monotone map fp32 -> uint32: larger float <=> larger key.
__device__ __forceinline__ uint32_t vote_key(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__global__ __launch_bounds__(kTopkThreads) void topk_kernel(TopkArgs a) {
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const ReqGeom geo = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;
  int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
  int32_t* sel_pos = a.sel_pos + (int64_t)b * a.sel_stride;
  const int L = geo.seq_len;

  auto emit = [&](int out_idx, int pos) {
    sel_pos[out_idx] = pos;
    sel[out_idx] = (int32_t)lookup_slot(tab, pos, a.page_size, a.page_shift, a.pool_rows);
  };

  if (geo.dense) {  // tr.py:377-378, 741-744: attend over every token
    for (int i = tid; i < L; i += kTopkThreads) emit(i, i);
    if (tid == 0) a.sel_len[b] = L;
    return;
  }

  const bool is_hit = a.hit && a.hit[b];
  const int k = is_hit ? min(a.cache_len[b], a.top_k) : geo.k;
  if (tid == 0) a.sel_len[b] = a.n_init + k + a.n_local;
  for (int i = tid; i < a.n_init; i += kTopkThreads) emit(i, i);
  for (int i = tid; i < a.n_local; i += kTopkThreads) emit(a.n_init + k + i, L - a.n_local + i);

  if (is_hit) {  // tr.py:419: reuse the cached positions
    const int32_t* cached = a.topk_cache + (int64_t)b * a.top_k;
    for (int i = tid; i < k; i += kTopkThreads) emit(a.n_init + i, cached[i]);
    return;
  }

  int n = geo.n;
  if (a.pool_kernel > 0 && (a.pool_kernel & 1) == 0) n -= 1;  // even kernel: one output fewer
  const float* votes = a.votes + (int64_t)b * a.vote_stride;

  __shared__ uint32_t hist[256];
  __shared__ uint32_t suffix[256];
  __shared__ uint32_t s_prefix, s_need;
  __shared__ uint32_t wave_gt[kTopkWaves], wave_eq[kTopkWaves];

  uint32_t prefix = 0, mask = 0, need = (uint32_t)k;
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += kTopkThreads) {
      const uint32_t key = vote_key(votes[i]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    // Inclusive suffix sums: suffix[d] = number of matching keys with digit >= d.
    if (tid < 256) suffix[tid] = hist[tid];
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      uint32_t add = 0;
      if (tid < 256 && tid + off < 256) add = suffix[tid + off];
      __syncthreads();
      if (tid < 256) suffix[tid] += add;
      __syncthreads();
    }
    if (tid < 256) {
      const uint32_t above = tid < 255 ? suffix[tid + 1] : 0u;
      if (suffix[tid] >= need && above < need) {  // exactly one digit satisfies this
        s_prefix = prefix | ((uint32_t)tid << shift);
        s_need = need - above;
      }
    }
    __syncthreads();
    prefix = s_prefix;
    need = s_need;
    mask |= 255u << shift;
    __syncthreads();
  }
  const uint32_t kth = prefix;     // key of the k-th largest vote
  const uint32_t need_eq = need;   // ties at kth to take, lowest position first

  int32_t* cache_out = a.topk_cache ? a.topk_cache + (int64_t)b * a.top_k : nullptr;
  uint32_t run_gt = 0, run_eq = 0;
  for (int base = 0; base < n; base += kTopkThreads) {
    const int i = base + tid;
    uint32_t key = 0;
    const bool in = i < n;
    if (in) key = vote_key(votes[i]);
    const bool gt = in && key > kth;
    const bool eq = in && key == kth;
    const uint64_t gt_mask = __ballot(gt), eq_mask = __ballot(eq);
    if (lane == 0) {
      wave_gt[wave] = __popcll(gt_mask);
      wave_eq[wave] = __popcll(eq_mask);
    }
    __syncthreads();
    uint32_t gt_before = 0, eq_before = 0, gt_total = 0, eq_total = 0;
#pragma unroll
    for (int w = 0; w < kTopkWaves; ++w) {
      const uint32_t g = wave_gt[w], e = wave_eq[w];
      if (w < wave) {
        gt_before += g;
        eq_before += e;
      }
      gt_total += g;
      eq_total += e;
    }
    const uint64_t below = (1ull << lane) - 1ull;
    gt_before += __popcll(gt_mask & below);
    eq_before += __popcll(eq_mask & below);
    const uint32_t eq_rank = run_eq + eq_before;
    if (gt || (eq && eq_rank < need_eq)) {
      const uint32_t out = run_gt + gt_before + min(eq_rank, need_eq);
      const int pos = a.n_init + i;
      emit(a.n_init + (int)out, pos);
      if (cache_out) cache_out[out] = pos;
    }
    run_gt += gt_total;
    run_eq += eq_total;
    __syncthreads();
  }
  if (tid == 0 && a.cache_len) a.cache_len[b] = k;
}

}  // namespace ts

using namespace ts;

extern "C" {

size_t ts_topk_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  (void)cfg;
  (void)batch;
  (void)max_seq_len;
  return 256;
}

int ts_topk_ragged(const ts_config* cfg, const ts_batch* bt, const float* votes,
                   int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                   int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                   void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  (void)workspace;
  (void)workspace_bytes;
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(votes && sel && sel_pos && sel_len, TS_EINVAL, "ts_topk_ragged: NULL tensor argument");
  const int max_sel = cfg->n_init + cfg->top_k + cfg->n_local;
  TS_REQUIRE(sel_stride >= max_sel, TS_EWORKSPACE, "sel_stride %lld < n_init+top_k+n_local = %d",
             (long long)sel_stride, max_sel);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  TS_REQUIRE(hit == nullptr || cache != nullptr, TS_EINVAL,
             "ts_topk_ragged: hit flags need the selection cache");
  if (cache)
    TS_REQUIRE(cache->topk_cache && cache->cache_len, TS_EINVAL,
               "ts_topk_ragged: selection cache has a NULL array");

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
  hipLaunchKernelGGL(topk_kernel, dim3((unsigned)bt->batch), dim3(kTopkThreads), 0,
                     (hipStream_t)stream, a);
  return check_launch("topk_kernel");
}

}  // extern "C"
