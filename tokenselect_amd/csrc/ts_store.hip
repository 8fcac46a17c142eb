// KV store and token-table append for a decode step
// (patched_radix_attention_store_kv_cache tr.py:844-854, add_k_cache tr.py:332-336).
#include "ts_pages.h"
#include "ts_store.h"

namespace ts {

// One workgroup per request: copies the new K and V rows (Hkv*128 bf16 each) to
// pool slot out_cache_loc[b], appends the slot to the request's table and bumps
// its length.  A full table (tr.py:334 asserts) or a slot outside the pool
// leaves the request untouched.
__global__ __launch_bounds__(256) void kv_store_kernel(const uint4* __restrict__ k,
                                                       const uint4* __restrict__ v,
                                                       const int32_t* __restrict__ loc,
                                                       uint4* __restrict__ k_pool,
                                                       uint4* __restrict__ v_pool, int64_t pool_rows,
                                                       int32_t* __restrict__ table,
                                                       int64_t table_stride,
                                                       int32_t* __restrict__ seq_lens,
                                                       int row_vec, int max_tokens) {
  const int b = blockIdx.x;
  // The new rows are asked for together with the slot and the length, not after them: the
  // kernel is two memory round trips long instead of three.
  const int first = threadIdx.x;
  uint4 k0 = make_uint4(0u, 0u, 0u, 0u), v0 = k0;
  if (first < row_vec) {
    k0 = k[(size_t)b * row_vec + first];
    v0 = v[(size_t)b * row_vec + first];
  }
  const int slot = loc[b];
  const int len = seq_lens[b];
  if (slot < 0 || slot >= pool_rows || len >= max_tokens) return;
  if (first < row_vec) {
    k_pool[(size_t)slot * row_vec + first] = k0;
    v_pool[(size_t)slot * row_vec + first] = v0;
  }
  for (int i = first + blockDim.x; i < row_vec; i += blockDim.x) {
    k_pool[(size_t)slot * row_vec + i] = k[(size_t)b * row_vec + i];
    v_pool[(size_t)slot * row_vec + i] = v[(size_t)b * row_vec + i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    table[(int64_t)b * table_stride + len] = slot;
    seq_lens[b] = len + 1;
  }
}

// Chunked prefill (tr.py:725-733): ts_store.h has the counted form's body, which the
// fingerprint launch of a chunk can also run on the side.
constexpr int kChunkRowsPerWg = 256 / kChunkThreadsPerRow;  // few workgroups, few counts on one word

template <bool COUNTED>
__global__ __launch_bounds__(256) void kv_store_chunk_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, const int32_t* __restrict__ loc,
    uint4* __restrict__ k_pool, uint4* __restrict__ v_pool, int64_t pool_rows,
    int32_t* __restrict__ table, int32_t* seq_len, int rows, int row_vec, int max_tokens) {
  ChunkStore cs{k, v, loc, k_pool, v_pool, pool_rows, table, seq_len, rows, row_vec, max_tokens, (int)gridDim.x};
  store_chunk_rows<COUNTED>(cs, (int)blockIdx.x, 256);
}

__global__ void seq_len_add_kernel(int32_t* seq_len, int rows, int max_tokens) {
  const int len = *seq_len + rows;
  *seq_len = len > max_tokens ? max_tokens : len;
}


// Paged form of kv_store_kernel: the slot comes from the request's table, or from a
// fresh page of the caller's free list when the length is a multiple of the page size
// (ts_pages.h).  One workgroup per request; nothing of the plan is written before the
// launch's last workgroup commits it.
__global__ __launch_bounds__(256) void kv_store_paged_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, uint4* __restrict__ k_pool,
    uint4* __restrict__ v_pool, uint32_t pool_rows, int32_t* table, int64_t table_stride,
    int32_t* seq_lens, int batch, int row_vec, int max_tokens, int page_shift, PagePool pool) {
  __shared__ uint32_t plan_slot, plan_ok;
  const int b = blockIdx.x, lane = threadIdx.x & 63;
  // (the new rows are asked for before the plan is made, not after)
  const int first = threadIdx.x;
  uint4 k0 = make_uint4(0u, 0u, 0u, 0u), v0 = k0;
  if (first < row_vec) {
    k0 = k[(size_t)b * row_vec + first];
    v0 = v[(size_t)b * row_vec + first];
  }
  if (threadIdx.x < 64)
    for_each_append(seq_lens, table, table_stride, batch, pool, page_shift, max_tokens, pool_rows,
                    lane, [&](int req, const AppendPlan& p) {
                      if (req == b) {
                        plan_slot = p.slot;
                        plan_ok = p.ok ? 1u : 0u;
                      }
                    });
  __syncthreads();
  if (plan_ok) {
    const size_t slot = plan_slot;
    if (first < row_vec) {
      k_pool[slot * row_vec + first] = k0;
      v_pool[slot * row_vec + first] = v0;
    }
    for (int i = first + blockDim.x; i < row_vec; i += blockDim.x) {
      k_pool[slot * row_vec + i] = k[(size_t)b * row_vec + i];
      v_pool[slot * row_vec + i] = v[(size_t)b * row_vec + i];
    }
  }
  __syncthreads();
  if (threadIdx.x < 64)
    commit_appends(seq_lens, table, table_stride, batch, pool, page_shift, max_tokens, pool_rows,
                   lane, gridDim.x);
}

// Where row r of a chunk goes when the request's table is paged: positions
// len .. len + rows - 1 fill the request's last page and then fresh pages from the
// top of the free list, in order.  The same arithmetic serves every workgroup and
// the commit.
struct ChunkPlan {
  int len, count;
  int first_new;  // first page index of the table that does not exist yet
  int stored;     // rows that fit the table and the pages left
  int taken;      // pages taken from the list
};

__device__ __forceinline__ ChunkPlan make_chunk_plan(const int32_t* seq_len, const PagePool& pool,
                                                     int rows, int max_tokens, int page_shift) {
  ChunkPlan c;
  c.len = min(max(*seq_len, 0), max_tokens);
  c.count = max(*pool.free_count, 0);
  const int page = 1 << page_shift;
  c.first_new = (c.len + page - 1) >> page_shift;
  const int fit = min(rows, max_tokens - c.len);
  const int wanted = fit > 0 ? ((c.len + fit - 1) >> page_shift) - c.first_new + 1 : 0;
  c.taken = min(max(wanted, 0), c.count);
  c.stored = c.taken == max(wanted, 0) ? fit : max(((c.first_new + c.taken) << page_shift) - c.len, 0);
  return c;
}

__global__ __launch_bounds__(256) void kv_store_chunk_paged_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, uint4* __restrict__ k_pool,
    uint4* __restrict__ v_pool, uint32_t pool_rows, int32_t* table, int32_t* seq_len, int rows,
    int row_vec, int max_tokens, int page_shift, PagePool pool) {
  const int r = blockIdx.x;
  const ChunkPlan c = make_chunk_plan(seq_len, pool, rows, max_tokens, page_shift);
  if (r < c.stored) {
    const int at = c.len + r;
    const int pg = at >> page_shift;
    const bool fresh = pg >= c.first_new;
    const int32_t page = fresh ? pool.free_pages[c.count - 1 - (pg - c.first_new)] : table[pg];
    uint32_t slot = ((uint32_t)page << page_shift) + (uint32_t)(at & ((1 << page_shift) - 1));
    slot = slot < pool_rows ? slot : pool_rows - 1;
    for (int i = threadIdx.x; i < row_vec; i += blockDim.x) {
      k_pool[(size_t)slot * row_vec + i] = k[(size_t)r * row_vec + i];
      v_pool[(size_t)slot * row_vec + i] = v[(size_t)r * row_vec + i];
    }
  }
  __syncthreads();
  if (threadIdx.x == 0 &&
      __hip_atomic_fetch_add(pool.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 ==
          gridDim.x) {
    for (int j = 0; j < c.taken; ++j) table[c.first_new + j] = pool.free_pages[c.count - 1 - j];
    *seq_len = c.len + c.stored;
    *pool.free_count = c.count - c.taken;
    __hip_atomic_store(pool.ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace ts

using namespace ts;

static int check_pool_arg(const ts_config* cfg, const int32_t* out_cache_loc, const ts_page_pool* pages,
                          const char* who) {
  if (pages) {
    TS_REQUIRE(pages->free_pages && pages->free_count && pages->ticket, TS_EINVAL,
               "%s: page pool has a NULL array", who);
    return TS_OK;
  }
  TS_REQUIRE(cfg->page_size == 1, TS_EINVAL,
             "%s: page_size %d needs a page pool (without one the caller's out_cache_loc is appended to "
             "a per-token table, page_size 1)",
             who, cfg->page_size);
  TS_REQUIRE(out_cache_loc != nullptr, TS_EINVAL, "%s: NULL out_cache_loc and no page pool", who);
  return TS_OK;
}

extern "C" int ts_kv_store(const ts_config* cfg, const void* k, const void* v,
                           const int32_t* out_cache_loc, const ts_page_pool* pages, void* k_pool,
                           void* v_pool, int64_t pool_rows, int32_t* table, int64_t table_stride,
                           int32_t* seq_lens, int32_t batch, int32_t max_tokens,
                           ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(k && v && k_pool && v_pool && table && seq_lens, TS_EINVAL,
             "ts_kv_store: NULL tensor argument");
  TS_REQUIRE_ALIGNED(k, 16, "k");
  TS_REQUIRE_ALIGNED(v, 16, "v");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_TRY(check_pool_arg(cfg, out_cache_loc, pages, "ts_kv_store"));
  TS_REQUIRE(batch >= 1 && pool_rows >= 1 && pool_rows <= 0x7fffffffLL && max_tokens >= 1, TS_EINVAL,
             "ts_kv_store: batch=%d pool_rows=%lld max_tokens=%d out of range", batch,
             (long long)pool_rows, max_tokens);
  TS_REQUIRE(batch == 1 || table_stride * (int64_t)cfg->page_size >= max_tokens, TS_EINVAL,
             "ts_kv_store: table_stride %lld x page_size %d < max_tokens %d", (long long)table_stride,
             cfg->page_size, max_tokens);
  const int row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  if (pages) {
    hipLaunchKernelGGL(kv_store_paged_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)k, (const uint4*)v, (uint4*)k_pool, (uint4*)v_pool,
                       (uint32_t)pool_rows, table, table_stride, seq_lens, batch, row_vec, max_tokens,
                       page_shift_of(cfg->page_size), page_pool_of(pages));
    return check_launch("kv_store_paged_kernel");
  }
  hipLaunchKernelGGL(kv_store_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)k, (const uint4*)v, out_cache_loc, (uint4*)k_pool, (uint4*)v_pool,
                     pool_rows, table, table_stride, seq_lens, row_vec, max_tokens);
  return check_launch("kv_store_kernel");
}

extern "C" int ts_kv_store_chunk(const ts_config* cfg, const void* k, const void* v,
                                 const int32_t* out_cache_loc, const ts_page_pool* pages, int32_t rows,
                                 void* k_pool, void* v_pool, int64_t pool_rows, int32_t* table,
                                 int32_t* seq_len, int32_t max_tokens, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(k && v && k_pool && v_pool && table && seq_len, TS_EINVAL,
             "ts_kv_store_chunk: NULL tensor argument");
  TS_REQUIRE_ALIGNED(k, 16, "k");
  TS_REQUIRE_ALIGNED(v, 16, "v");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_TRY(check_pool_arg(cfg, out_cache_loc, pages, "ts_kv_store_chunk"));
  TS_REQUIRE(rows >= 0 && pool_rows >= 1 && pool_rows <= 0x7fffffffLL && max_tokens >= 1, TS_EINVAL,
             "ts_kv_store_chunk: rows=%d pool_rows=%lld max_tokens=%d out of range", rows,
             (long long)pool_rows, max_tokens);
  if (rows == 0) return TS_OK;
  const int row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  if (pages) {
    hipLaunchKernelGGL(kv_store_chunk_paged_kernel, dim3((unsigned)rows), dim3(256), 0,
                       (hipStream_t)stream, (const uint4*)k, (const uint4*)v, (uint4*)k_pool,
                       (uint4*)v_pool, (uint32_t)pool_rows, table, seq_len, rows, row_vec, max_tokens,
                       page_shift_of(cfg->page_size), page_pool_of(pages));
    return check_launch("kv_store_chunk_paged_kernel");
  }
  const unsigned wgs = (unsigned)ceil_div(rows, kChunkRowsPerWg);
  if (wgs <= (unsigned)kChunkCountedWgs && max_tokens <= kLenMask) {
    hipLaunchKernelGGL(kv_store_chunk_kernel<true>, dim3(wgs), dim3(256), 0, (hipStream_t)stream,
                       (const uint4*)k, (const uint4*)v, out_cache_loc, (uint4*)k_pool, (uint4*)v_pool,
                       pool_rows, table, seq_len, rows, row_vec, max_tokens);
    return check_launch("kv_store_chunk_kernel");
  }
  hipLaunchKernelGGL(kv_store_chunk_kernel<false>, dim3(wgs), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)k, (const uint4*)v, out_cache_loc, (uint4*)k_pool, (uint4*)v_pool,
                     pool_rows, table, seq_len, rows, row_vec, max_tokens);
  TS_TRY(check_launch("kv_store_chunk_kernel"));
  hipLaunchKernelGGL(seq_len_add_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, seq_len, rows,
                     max_tokens);
  return check_launch("seq_len_add_kernel");
}
