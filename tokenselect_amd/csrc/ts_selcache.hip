// Selection cache decision (tr.py:394-401, 416-421): compare the query
// fingerprint with the one cached at the last miss; reuse the cached top-k on a
// hit.  The decision stays on the device as a flag that the later kernels read,
// so a decode step needs no host synchronisation.
#include "ts_common.h"

namespace ts {

struct SelCacheArgs {
  const uint16_t* qf;  // [B, H*D] bf16
  uint16_t* q_cache;   // [B, H*D] bf16
  const int32_t* cache_len;
  int64_t* counters;
  float threshold;
  const int32_t* seq_lens;
  const int32_t* k_per_req;
  int n_init, n_local, top_k, max_seq_len;
  int dim;  // H*D
  int32_t* hit;
  // A call that repeats the step's previous one after a give-up: requests whose entry of
  // gave_up_len is negative were selecting when it happened and their cache entry is not
  // valid (a miss whatever the cache holds); the counters have advanced already.
  const int32_t* gave_up_len;  // or NULL
};

constexpr int kSelCacheMaxVec = 4;  // 16-byte pieces per thread: 64 heads x 128 / 8 / 256

__global__ __launch_bounds__(256) void selcache_kernel(SelCacheArgs a) {
  const int b = blockIdx.x;
  const ReqGeom geo = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  if (geo.dense) {  // tr.py:377-378 returns before the cache is consulted
    if (threadIdx.x == 0) a.hit[b] = 0;
    return;
  }
  const uint16_t* q = a.qf + (size_t)b * a.dim;
  uint16_t* qc = a.q_cache + (size_t)b * a.dim;
  const bool have = a.cache_len[b] > 0 &&  // is_first_query is false
                    !(a.gave_up_len && a.gave_up_len[b] < 0);

  // dim = H * 128 elements, at most kMaxVec 16-byte pieces per thread, all requested at
  // once (one piece per thread and pass: a loop of dependent 2-byte loads took 8 us).
  constexpr int kMaxVec = kSelCacheMaxVec;
  const int pieces = a.dim >> 3;
  uint4 qv[kMaxVec], cv[kMaxVec];
#pragma unroll
  for (int j = 0; j < kMaxVec; ++j) {
    const int i = threadIdx.x + 256 * j;
    qv[j] = i < pieces ? ((const uint4*)q)[i] : make_uint4(0u, 0u, 0u, 0u);
    cv[j] = (have && i < pieces) ? ((const uint4*)qc)[i] : make_uint4(0u, 0u, 0u, 0u);
  }
  float dot = 0.f, nq = 0.f, nc = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxVec; ++j) {
    const uint32_t xs[4] = {qv[j].x, qv[j].y, qv[j].z, qv[j].w};
    const uint32_t ys[4] = {cv[j].x, cv[j].y, cv[j].z, cv[j].w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float x0 = bf16_lo(xs[e]), x1 = bf16_hi(xs[e]), y0 = bf16_lo(ys[e]), y1 = bf16_hi(ys[e]);
      dot += x0 * y0 + x1 * y1;
      nq += x0 * x0 + x1 * x1;
      nc += y0 * y0 + y1 * y1;
    }
  }
  __shared__ float red[3][4];
  dot = row16_sum(dot);
  nq = row16_sum(nq);
  nc = row16_sum(nc);
  dot += __shfl_xor(dot, 16); nq += __shfl_xor(nq, 16); nc += __shfl_xor(nc, 16);
  dot += __shfl_xor(dot, 32); nq += __shfl_xor(nq, 32); nc += __shfl_xor(nc, 32);
  if ((threadIdx.x & 63) == 0) {
    red[0][threadIdx.x >> 6] = dot;
    red[1][threadIdx.x >> 6] = nq;
    red[2][threadIdx.x >> 6] = nc;
  }
  __syncthreads();
  dot = red[0][0] + red[0][1] + red[0][2] + red[0][3];
  nq = red[1][0] + red[1][1] + red[1][2] + red[1][3];
  nc = red[2][0] + red[2][1] + red[2][2] + red[2][3];
  const float cosine = dot / fmaxf(sqrtf(nq) * sqrtf(nc), 1e-8f);
  const bool is_hit = have && !(cosine < a.threshold);  // tr.py:395-401
  if (!is_hit) {  // tr.py:416
#pragma unroll
    for (int j = 0; j < kMaxVec; ++j) {
      const int i = threadIdx.x + 256 * j;
      if (i < pieces) ((uint4*)qc)[i] = qv[j];
    }
  }
  if (threadIdx.x == 0) {
    a.hit[b] = is_hit ? 1 : 0;
    if (a.gave_up_len == nullptr) {
      if (is_hit) a.counters[2 * b] += 1;  // skip_count, tr.py:420
      a.counters[2 * b + 1] += 1;          // retrieval_count, tr.py:421
    }
  }
}

int launch_selcache(const ts_config* cfg, const ts_batch* bt, const void* qf, const ts_selcache* cache,
                    int32_t* hit, const int32_t* gave_up_len, hipStream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(qf && cache && hit, TS_EINVAL, "ts_selcache_step: NULL argument");
  TS_REQUIRE(cache->q_cache && cache->topk_cache && cache->cache_len && cache->counters, TS_EINVAL,
             "ts_selcache_step: selection cache has a NULL array");
  SelCacheArgs a;
  a.qf = (const uint16_t*)qf;
  a.q_cache = (uint16_t*)cache->q_cache;
  a.cache_len = cache->cache_len;
  a.counters = cache->counters;
  a.threshold = cache->threshold;
  a.seq_lens = bt->seq_lens;
  a.k_per_req = bt->k_per_req;
  a.n_init = cfg->n_init;
  a.n_local = cfg->n_local;
  a.top_k = cfg->top_k;
  a.max_seq_len = bt->max_seq_len;
  a.dim = cfg->num_heads * cfg->head_dim;
  TS_REQUIRE(a.dim % 8 == 0 && a.dim <= kSelCacheMaxVec * 256 * 8, TS_ESHAPE,
             "ts_selcache_step: %d query elements per request (at most %d)", a.dim, kSelCacheMaxVec * 256 * 8);
  a.hit = hit;
  a.gave_up_len = gave_up_len;
  hipLaunchKernelGGL(selcache_kernel, dim3((unsigned)bt->batch), dim3(256), 0, stream, a);
  return check_launch("selcache_kernel");
}

}  // namespace ts

using namespace ts;

extern "C" int ts_selcache_step(const ts_config* cfg, const ts_batch* bt, const void* qf,
                                const ts_selcache* cache, int32_t* hit, ts_stream_t stream) {
  return launch_selcache(cfg, bt, qf, cache, hit, nullptr, (hipStream_t)stream);
}
