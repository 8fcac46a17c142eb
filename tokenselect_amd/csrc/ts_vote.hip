// Soft vote: per-head softmax over the candidates summed over heads (tr.py:361),
// and the optional max-pool smoothing of the votes (tr.py:366-369).
//
// Scores arrive tile-major from the scoring pass: scores[b][tile][slot][16] with
// head slot = kvh*G + g (see ts_score.hip); a thread owns one candidate and walks
// the H slots of its tile, so a wavefront reads four contiguous 16*H*4-byte tiles.
#include "ts_topk.h"

namespace ts {

constexpr int kMaxHeads = 128;

struct VoteArgs {
  const float* scores;
  int64_t score_stride;   // token slots per request (multiple of 16)
  const float* partials;  // [B,H,nchunks,2] from the scoring pass, by head
  int nchunks, tokens_per_block;
  float* stats;           // [B,H,2] merged (max, sum exp), by head
  const int32_t* seq_lens;
  const int32_t* k_per_req;
  const int32_t* skip;
  int n_init, n_local, top_k, num_heads, num_kv_heads, head_map, max_seq_len;
  float* votes;
  int64_t vote_stride;
  // Per-request top-k workspace whose first-level histogram the vote kernel fills
  // (zero at launch), or NULL.
  uint32_t* hist_ws;
  size_t hist_ws_stride;
};

// Merge the per-workgroup softmax partials of one (request, head).
__global__ __launch_bounds__(64) void stats_merge_kernel(VoteArgs a) {
  const int h = blockIdx.x, b = blockIdx.y;
  if (a.skip && a.skip[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  if (geo.n <= 0) return;
  const int chunks = (geo.n + a.tokens_per_block - 1) / a.tokens_per_block;
  const float* p = a.partials + ((size_t)b * a.num_heads + h) * a.nchunks * 2;
  float m = kNegBig, l = 0.f;
  for (int c = threadIdx.x; c < chunks; c += 64) softmax_merge(m, l, p[2 * c], p[2 * c + 1]);
  row16_softmax_merge(m, l);
  softmax_merge(m, l, __shfl_xor(m, 16), __shfl_xor(l, 16));
  softmax_merge(m, l, __shfl_xor(m, 32), __shfl_xor(l, 32));
  if (threadIdx.x == 0) {
    a.stats[((size_t)b * a.num_heads + h) * 2] = m;
    a.stats[((size_t)b * a.num_heads + h) * 2 + 1] = l;
  }
}

// A thread owns four candidates, 256 apart; fp32 sum over the head slots in slot
// order.  With a top-k workspace attached the workgroup also counts its votes into the
// first-level histogram of the selection (top 11 key bits) and adds its occupied bins
// to the request's histogram at the end.
template <int kPerThread>  // candidates per thread: a workgroup owns 256 * kPerThread
__global__ __launch_bounds__(256) void vote_kernel(VoteArgs a) {
  constexpr int kVoteSlice = 256 * kPerThread;
  const int b = blockIdx.y;
  if (a.skip && a.skip[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int block_lo = blockIdx.x * kVoteSlice;
  if (block_lo >= geo.n) return;

  __shared__ float s_max[kMaxHeads];
  __shared__ float s_rz[kMaxHeads];
  __shared__ uint32_t lh[kTopkBins];
  const int H = a.num_heads;
  const int group = H / a.num_kv_heads;
  for (int slot = threadIdx.x; slot < H; slot += 256) {
    const int kvh = slot / group, g = slot % group;
    const int h = a.head_map == TS_HEADMAP_MOD ? kvh + a.num_kv_heads * g : slot;
    s_max[slot] = a.stats[((size_t)b * H + h) * 2];
    s_rz[slot] = 1.0f / a.stats[((size_t)b * H + h) * 2 + 1];
  }
  if (a.hist_ws)
    for (int i = threadIdx.x; i < kTopkBins; i += 256) lh[i] = 0u;
  __syncthreads();

  float c[kPerThread];
  const float* p[kPerThread];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int t = min(block_lo + j * 256 + (int)threadIdx.x, geo.n - 1);  // clamped: no branch
    p[j] = a.scores + ((size_t)b * a.score_stride + (size_t)(t & ~15)) * H + (t & 15);
    c[j] = 0.f;
  }
  int slot = 0;
  for (; slot + 4 <= H; slot += 4) {
    float s[kPerThread][4];
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) s[j][i] = p[j][(slot + i) * 16];
#pragma unroll
    for (int j = 0; j < kPerThread; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) c[j] += __expf(s[j][i] - s_max[slot + i]) * s_rz[slot + i];
  }
  for (; slot < H; ++slot)
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) c[j] += __expf(p[j][slot * 16] - s_max[slot]) * s_rz[slot];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int t = block_lo + j * 256 + (int)threadIdx.x;
    if (t < geo.n) {
      a.votes[(size_t)b * a.vote_stride + t] = c[j];
      if (a.hist_ws) atomicAdd(&lh[key_bin0(vote_key(c[j]))], 1u);
    }
  }
  if (a.hist_ws) {
    __syncthreads();
    uint32_t* hist0 = topk_ws(a.hist_ws, a.hist_ws_stride, b) + kTopkHist0;
    for (int i = threadIdx.x; i < kTopkBins; i += 256)
      if (lh[i]) atomicAdd(&hist0[i], lh[i]);
  }
}

struct PoolArgs {
  const float* votes;
  float* pooled;
  int64_t vote_stride, pooled_stride;
  const int32_t* seq_lens;
  const int32_t* k_per_req;
  const int32_t* skip;
  int n_init, n_local, top_k, kernel, max_seq_len;
};

// max_pool1d(kernel, stride 1, padding (kernel-1)/2) over the n votes: output t
// covers inputs [t - pad, t - pad + kernel) clipped to [0, n); an even kernel
// yields n-1 outputs (tr.py:366-369).
__global__ __launch_bounds__(256) void pool_kernel(PoolArgs a) {
  const int b = blockIdx.y;
  if (a.skip && a.skip[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int pad = (a.kernel - 1) / 2;
  const int n_out = geo.n + 2 * pad - a.kernel + 1;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= n_out) return;
  const float* v = a.votes + (size_t)b * a.vote_stride;
  const int lo = max(t - pad, 0), hi = min(t - pad + a.kernel, geo.n);
  float m = v[lo];
  for (int i = lo + 1; i < hi; ++i) m = fmaxf(m, v[i]);
  a.pooled[(size_t)b * a.pooled_stride + t] = m;
}

int launch_pool(const ts_config* cfg, const ts_batch* bt, const float* votes, int64_t vote_stride,
                float* pooled, int64_t pooled_stride, const int32_t* skip, hipStream_t stream) {
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  if (max_n <= 0) return TS_OK;
  PoolArgs p;
  p.votes = votes;
  p.pooled = pooled;
  p.vote_stride = vote_stride;
  p.pooled_stride = pooled_stride;
  p.seq_lens = bt->seq_lens;
  p.k_per_req = bt->k_per_req;
  p.skip = skip;
  p.n_init = cfg->n_init;
  p.n_local = cfg->n_local;
  p.top_k = cfg->top_k;
  p.max_seq_len = bt->max_seq_len;
  p.kernel = cfg->pool_kernel;
  hipLaunchKernelGGL(pool_kernel, dim3((unsigned)ceil_div(max_n, 256), (unsigned)bt->batch), dim3(256),
                     0, stream, p);
  return check_launch("pool_kernel");
}

int launch_vote(const ts_config* cfg, const ts_batch* bt, const float* scores, int64_t score_stride,
                const float* partials, const int32_t* skip, float* stats, float* votes,
                float* pooled, int64_t vote_stride, uint32_t* hist_ws, size_t hist_ws_stride,
                hipStream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(scores && partials && stats && votes, TS_EINVAL, "ts_vote: NULL tensor argument");
  TS_REQUIRE(cfg->num_heads <= kMaxHeads, TS_ESHAPE, "num_heads %d > %d", cfg->num_heads, kMaxHeads);
  TS_REQUIRE(cfg->pool_kernel <= 0 || pooled != nullptr, TS_EINVAL,
             "ts_vote: pool_kernel %d needs a pooled buffer", cfg->pool_kernel);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(score_stride >= max_n && score_stride % 16 == 0 && vote_stride >= max_n, TS_EWORKSPACE,
             "ts_vote: stride (%lld, %lld) < max candidates %d or score_stride not a multiple of 16",
             (long long)score_stride, (long long)vote_stride, max_n);
  if (max_n <= 0) return TS_OK;

  VoteArgs a;
  a.scores = scores;
  a.score_stride = score_stride;
  a.partials = partials;
  a.tokens_per_block = score_tokens_per_block((int64_t)bt->batch * bt->max_seq_len, cfg->num_heads);
  a.nchunks = (int)ceil_div(bt->max_seq_len, a.tokens_per_block);
  a.stats = stats;
  a.seq_lens = bt->seq_lens;
  a.k_per_req = bt->k_per_req;
  a.skip = skip;
  a.n_init = cfg->n_init;
  a.n_local = cfg->n_local;
  a.top_k = cfg->top_k;
  a.max_seq_len = bt->max_seq_len;
  a.num_heads = cfg->num_heads;
  a.num_kv_heads = cfg->num_kv_heads;
  a.head_map = cfg->head_map;
  a.votes = votes;
  a.vote_stride = vote_stride;
  a.hist_ws = cfg->pool_kernel > 0 ? nullptr : hist_ws;  // the selection sees the pooled votes
  a.hist_ws_stride = hist_ws_stride;
  hipLaunchKernelGGL(stats_merge_kernel, dim3((unsigned)cfg->num_heads, (unsigned)bt->batch), dim3(64),
                     0, stream, a);
  TS_TRY(check_launch("stats_merge_kernel"));
  // Four candidates per thread: the workgroups' histogram flushes (a scan of 2048 LDS
  // bins and an atomic per occupied one) cost more than the parallelism of smaller
  // workgroup ranges brings, also at 128K candidates.
  hipLaunchKernelGGL(vote_kernel<4>, dim3((unsigned)ceil_div(max_n, 1024), (unsigned)bt->batch),
                     dim3(256), 0, stream, a);
  TS_TRY(check_launch("vote_kernel"));

  if (cfg->pool_kernel > 0)
    TS_TRY(launch_pool(cfg, bt, votes, vote_stride, pooled, vote_stride, skip, stream));
  return TS_OK;
}

}  // namespace ts

using namespace ts;

extern "C" int ts_vote(const ts_config* cfg, const ts_batch* bt, const float* scores,
                       int64_t score_stride, const float* partials, const int32_t* skip,
                       float* stats, float* votes, float* pooled, int64_t vote_stride,
                       ts_stream_t stream) {
  return launch_vote(cfg, bt, scores, score_stride, partials, skip, stats, votes, pooled,
                     vote_stride, nullptr, 0, (hipStream_t)stream);
}
