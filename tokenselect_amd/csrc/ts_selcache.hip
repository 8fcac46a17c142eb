// Selection cache decision (tr.py:394-401, 416-421): compare the query
// fingerprint with the one cached at the last miss; reuse the cached top-k on a
// hit.  The decision stays on the device as a flag that the later kernels read,
// so a decode step needs no host synchronisation.
#include <algorithm>

#include "ts_common.h"
#include "ts_pages.h"

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
    cv[j] = i < pieces ? ((const uint4*)qc)[i] : make_uint4(0u, 0u, 0u, 0u);  // (valid or not: see `have`)
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

// The fingerprint rotation of a decode step (rope_apply_kernel, one row per request) and the
// cache decision in one launch: the two sit on the step's dependent chain, and a launch
// costs about as much as either of them.  Workgroup b rotates request b's query (bit for
// bit as rope_apply_kernel does), writes the fingerprint and takes the decision from the
// rounded values it has just written; the workgroups beyond the batch clear.
// A thread owns units of two 16-byte pieces: dims [8u, 8u + 8) of a head and their rotation
// partners 64 dims further on.
__global__ __launch_bounds__(256) void rope_selcache_kernel(const uint16_t* __restrict__ x,
                                                           uint16_t* __restrict__ qf_out,
                                                           const float* __restrict__ cos_row,
                                                           const float* __restrict__ sin_row,
                                                           SelCacheArgs a, int batch, ZeroSet zero,
                                                           StepStore st) {
#pragma clang fp contract(off)
  const int b = blockIdx.x;
  if (b >= batch) {  // the clearing is the other workgroups' job: the decision is a chain of its own
    clear_regions(zero, (int64_t)(b - batch) * 256 + threadIdx.x, (int64_t)((int)gridDim.x - batch) * 256);
    return;
  }
  constexpr int kMaxUnits = kSelCacheMaxVec / 2;
  const int units = a.dim >> 4;  // (heads x 8)
  // With a token to store (st.k): this workgroup stores request b's rows and appends the slot
  // exactly as kv_store_kernel does, and decides with the length after the append, which it
  // knows without reading it back.
  // (One thread reads the length and hands it round: the append below rewrites the word.)
  __shared__ int len_before;
  if (threadIdx.x == 0) len_before = a.seq_lens[b];
  __syncthreads();
  int len_now = len_before;
  // The rows are asked for here and written at the kernel's end: a store waits for its data,
  // and every instruction behind it (the query's loads among them) would wait with it.
  const int first = threadIdx.x;
  uint4 k0 = make_uint4(0u, 0u, 0u, 0u), v0 = k0;
  int store_slot = -1;
  const bool paged = st.k != nullptr && st.free_pages != nullptr;
  const PagePool pool{st.free_pages, st.free_count, st.ticket};
  if (st.k != nullptr) {
    if (first < st.row_vec) {
      k0 = st.k[(size_t)b * st.row_vec + first];
      v0 = st.v[(size_t)b * st.row_vec + first];
    }
    if (paged) {
      // The plan of the whole batch from the snapshot that no workgroup modifies before the
      // launch's last one commits it (at the end of this kernel); this request's part of it.
      __shared__ int plan_slot;
      if (threadIdx.x == 0) plan_slot = -1;
      __syncthreads();
      if (threadIdx.x < 64)
        for_each_append(st.seq_lens, st.table, st.table_stride, batch, pool, st.page_shift, st.max_tokens,
                        (uint32_t)st.pool_rows, (int)threadIdx.x, [&](int req, const AppendPlan& p) {
                          if (req == b && p.ok) plan_slot = (int)p.slot;
                        });
      __syncthreads();
      store_slot = plan_slot;
      if (store_slot >= 0) len_now += 1;
    } else {
      const int slot = st.loc[b];
      if (slot >= 0 && slot < st.pool_rows && len_now < st.max_tokens) {
        store_slot = slot;
        if (threadIdx.x == 0) {
          st.table[(int64_t)b * st.table_stride + len_now] = slot;
          st.seq_lens[b] = len_now + 1;
        }
        len_now += 1;
      }
    }
  }
  auto store_rows = [&]() {
    if (store_slot >= 0) {
      if (first < st.row_vec) {
        st.k_pool[(size_t)store_slot * st.row_vec + first] = k0;
        st.v_pool[(size_t)store_slot * st.row_vec + first] = v0;
      }
      for (int i = first + 256; i < st.row_vec; i += 256) {
        st.k_pool[(size_t)store_slot * st.row_vec + i] = st.k[(size_t)b * st.row_vec + i];
        st.v_pool[(size_t)store_slot * st.row_vec + i] = st.v[(size_t)b * st.row_vec + i];
      }
    }
    // (the workgroups of the requests are the launch that stores: the last of them commits)
    if (paged && threadIdx.x < 64)
      commit_appends(st.seq_lens, st.table, st.table_stride, batch, pool, st.page_shift, st.max_tokens,
                     (uint32_t)st.pool_rows, (int)threadIdx.x, (uint32_t)batch);
  };
  ReqGeom geo;
  {
    geo.seq_len = min(max(len_now, 0), a.max_seq_len);
    const int kk = a.k_per_req ? a.k_per_req[b] : a.top_k;
    geo.k = kk < 0 ? 0 : (kk > a.top_k ? a.top_k : kk);
    geo.dense = (a.n_init + geo.k + a.n_local >= geo.seq_len);
    geo.n = geo.dense ? 0 : geo.seq_len - a.n_init - a.n_local;
  }
  const uint16_t* q = x + (size_t)b * a.dim;
  uint16_t* qo = qf_out + (size_t)b * a.dim;
  uint16_t* qc = a.q_cache + (size_t)b * a.dim;
  const bool have = !geo.dense && a.cache_len[b] > 0 && !(a.gave_up_len && a.gave_up_len[b] < 0);
  uint4 lo_raw[kMaxUnits], hi_raw[kMaxUnits], clo[kMaxUnits], chi[kMaxUnits];
  float4 c_lo[kMaxUnits][2], s_lo[kMaxUnits][2], c_hi[kMaxUnits][2], s_hi[kMaxUnits][2];
#pragma unroll
  for (int j = 0; j < kMaxUnits; ++j) {
    const int u = threadIdx.x + 256 * j;
    const bool live = u < units;
    const int head = u >> 3, d0 = (u & 7) * 8;  // dims d0 .. d0 + 7 and d0 + 64 .. d0 + 71
    const size_t at = (size_t)head * kHeadDim + d0;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    lo_raw[j] = live ? *(const uint4*)(q + at) : zero4;
    hi_raw[j] = live ? *(const uint4*)(q + at + 64) : zero4;
    // (the cached query is asked for whether or not the entry is valid: waiting for the
    // request's length and the cache's state first would be a round trip of its own)
    clo[j] = live ? *(const uint4*)(qc + at) : zero4;
    chi[j] = live ? *(const uint4*)(qc + at + 64) : zero4;
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      c_lo[j][v] = *(const float4*)(cos_row + d0 + 4 * v);
      s_lo[j][v] = *(const float4*)(sin_row + d0 + 4 * v);
      c_hi[j][v] = *(const float4*)(cos_row + 64 + d0 + 4 * v);
      s_hi[j][v] = *(const float4*)(sin_row + 64 + d0 + 4 * v);
    }
  }
  float dot = 0.f, nq = 0.f, nc = 0.f;
  uint4 out_lo[kMaxUnits], out_hi[kMaxUnits];
#pragma unroll
  for (int j = 0; j < kMaxUnits; ++j) {
    const uint32_t xl[4] = {lo_raw[j].x, lo_raw[j].y, lo_raw[j].z, lo_raw[j].w};
    const uint32_t xh[4] = {hi_raw[j].x, hi_raw[j].y, hi_raw[j].z, hi_raw[j].w};
    const uint32_t yl[4] = {clo[j].x, clo[j].y, clo[j].z, clo[j].w};
    const uint32_t yh[4] = {chi[j].x, chi[j].y, chi[j].z, chi[j].w};
    const float cl[8] = {c_lo[j][0].x, c_lo[j][0].y, c_lo[j][0].z, c_lo[j][0].w,
                         c_lo[j][1].x, c_lo[j][1].y, c_lo[j][1].z, c_lo[j][1].w};
    const float sl[8] = {s_lo[j][0].x, s_lo[j][0].y, s_lo[j][0].z, s_lo[j][0].w,
                         s_lo[j][1].x, s_lo[j][1].y, s_lo[j][1].z, s_lo[j][1].w};
    const float ch[8] = {c_hi[j][0].x, c_hi[j][0].y, c_hi[j][0].z, c_hi[j][0].w,
                         c_hi[j][1].x, c_hi[j][1].y, c_hi[j][1].z, c_hi[j][1].w};
    const float sh[8] = {s_hi[j][0].x, s_hi[j][0].y, s_hi[j][0].z, s_hi[j][0].w,
                         s_hi[j][1].x, s_hi[j][1].y, s_hi[j][1].z, s_hi[j][1].w};
    uint32_t ol[4], oh[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint16_t rl[2], rh[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const float x1 = t ? bf16_hi(xl[e]) : bf16_lo(xl[e]);
        const float x2 = t ? bf16_hi(xh[e]) : bf16_lo(xh[e]);
        const int i = 2 * e + t;
        // out = x * cos + rotate_half(x) * sin, products and sum rounded one by one
        rl[t] = f32_to_bf16(x1 * cl[i] + (-x2) * sl[i]);
        rh[t] = f32_to_bf16(x2 * ch[i] + x1 * sh[i]);
        const float ql = bf16_to_f32(rl[t]), qh = bf16_to_f32(rh[t]);
        const float y1 = t ? bf16_hi(yl[e]) : bf16_lo(yl[e]);
        const float y2 = t ? bf16_hi(yh[e]) : bf16_lo(yh[e]);
        dot += ql * y1 + qh * y2;
        nq += ql * ql + qh * qh;
        nc += y1 * y1 + y2 * y2;
      }
      ol[e] = (uint32_t)rl[0] | ((uint32_t)rl[1] << 16);
      oh[e] = (uint32_t)rh[0] | ((uint32_t)rh[1] << 16);
    }
    out_lo[j] = make_uint4(ol[0], ol[1], ol[2], ol[3]);
    out_hi[j] = make_uint4(oh[0], oh[1], oh[2], oh[3]);
    const int u = threadIdx.x + 256 * j;
    if (u < units) {
      const size_t at = (size_t)(u >> 3) * kHeadDim + (u & 7) * 8;
      *(uint4*)(qo + at) = out_lo[j];
      *(uint4*)(qo + at + 64) = out_hi[j];
    }
  }
  if (geo.dense) {  // tr.py:377-378 returns before the cache is consulted
    if (threadIdx.x == 0) a.hit[b] = 0;
    store_rows();
    return;
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
    for (int j = 0; j < kMaxUnits; ++j) {
      const int u = threadIdx.x + 256 * j;
      if (u < units) {
        const size_t at = (size_t)(u >> 3) * kHeadDim + (u & 7) * 8;
        *(uint4*)(qc + at) = out_lo[j];
        *(uint4*)(qc + at + 64) = out_hi[j];
      }
    }
  }
  if (threadIdx.x == 0) {
    a.hit[b] = is_hit ? 1 : 0;
    if (a.gave_up_len == nullptr) {
      if (is_hit) a.counters[2 * b] += 1;  // skip_count, tr.py:420
      a.counters[2 * b + 1] += 1;          // retrieval_count, tr.py:421
    }
  }
  store_rows();
}

static int fill_selcache_args(const ts_config* cfg, const ts_batch* bt, const void* qf,
                              const ts_selcache* cache, int32_t* hit, const int32_t* gave_up_len,
                              SelCacheArgs* out) {
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
  *out = a;
  return TS_OK;
}

int launch_selcache(const ts_config* cfg, const ts_batch* bt, const void* qf, const ts_selcache* cache,
                    int32_t* hit, const int32_t* gave_up_len, hipStream_t stream) {
  SelCacheArgs a;
  TS_TRY(fill_selcache_args(cfg, bt, qf, cache, hit, gave_up_len, &a));
  hipLaunchKernelGGL(selcache_kernel, dim3((unsigned)bt->batch), dim3(256), 0, stream, a);
  return check_launch("selcache_kernel");
}

int launch_rope_selcache(const ts_config* cfg, const ts_batch* bt, const void* q, void* qf,
                         const float* q_cos, const float* q_sin, const ts_selcache* cache, int32_t* hit,
                         const int32_t* gave_up_len, const ZeroSet& zero, hipStream_t stream,
                         const StepStore* store) {
  SelCacheArgs a;
  TS_TRY(fill_selcache_args(cfg, bt, qf, cache, hit, gave_up_len, &a));
  StepStore st{};
  if (store) st = *store;
  TS_REQUIRE(!zero.overflow, TS_EINVAL, "internal: more than %d regions to clear in one launch", kZeroRegions);
  TS_REQUIRE_ALIGNED(q_cos, 16, "q_cos");
  TS_REQUIRE_ALIGNED(q_sin, 16, "q_sin");
  const int64_t blocks = bt->batch + std::max<int64_t>(1, ceil_div(zero.total(), 1024));
  hipLaunchKernelGGL(rope_selcache_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                     (const uint16_t*)q, (uint16_t*)qf, q_cos, q_sin, a, bt->batch, zero, st);
  return check_launch("rope_selcache_kernel");
}

}  // namespace ts

using namespace ts;

extern "C" int ts_selcache_step(const ts_config* cfg, const ts_batch* bt, const void* qf,
                                const ts_selcache* cache, int32_t* hit, ts_stream_t stream) {
  return launch_selcache(cfg, bt, qf, cache, hit, nullptr, (hipStream_t)stream);
}
