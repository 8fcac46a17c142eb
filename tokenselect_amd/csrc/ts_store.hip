// KV store and token-table append for a decode step
// (patched_radix_attention_store_kv_cache tr.py:844-854, add_k_cache tr.py:332-336).
#include "ts_common.h"

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
  const int slot = loc[b];
  const int len = seq_lens[b];
  if (slot < 0 || slot >= pool_rows || len >= max_tokens) return;
  for (int i = threadIdx.x; i < row_vec; i += blockDim.x) {
    k_pool[(size_t)slot * row_vec + i] = k[(size_t)b * row_vec + i];
    v_pool[(size_t)slot * row_vec + i] = v[(size_t)b * row_vec + i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    table[(int64_t)b * table_stride + len] = slot;
    seq_lens[b] = len + 1;
  }
}

// Chunked prefill (tr.py:725-733): workgroup r copies row r of the chunk to pool
// slot loc[r] and writes table[len + r]; a second one-thread launch bumps the
// length, so that every workgroup of the first reads the same old length.  Rows
// that would not fit the table are dropped; slots are clamped to the pool.
__global__ __launch_bounds__(256) void kv_store_chunk_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, const int32_t* __restrict__ loc,
    uint4* __restrict__ k_pool, uint4* __restrict__ v_pool, int64_t pool_rows,
    int32_t* __restrict__ table, const int32_t* __restrict__ seq_len, int row_vec, int max_tokens) {
  const int r = blockIdx.x;
  const int at = *seq_len + r;
  if (at < 0 || at >= max_tokens) return;
  int64_t slot = loc[r];
  slot = slot < 0 ? 0 : (slot >= pool_rows ? pool_rows - 1 : slot);
  for (int i = threadIdx.x; i < row_vec; i += blockDim.x) {
    k_pool[(size_t)slot * row_vec + i] = k[(size_t)r * row_vec + i];
    v_pool[(size_t)slot * row_vec + i] = v[(size_t)r * row_vec + i];
  }
  if (threadIdx.x == 0) table[at] = (int32_t)slot;
}

__global__ void seq_len_add_kernel(int32_t* seq_len, int rows, int max_tokens) {
  const int len = *seq_len + rows;
  *seq_len = len > max_tokens ? max_tokens : len;
}

}  // namespace ts

using namespace ts;

extern "C" int ts_kv_store(const ts_config* cfg, const void* k, const void* v,
                           const int32_t* out_cache_loc, void* k_pool, void* v_pool,
                           int64_t pool_rows, int32_t* table, int64_t table_stride,
                           int32_t* seq_lens, int32_t batch, int32_t max_tokens,
                           ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(k && v && out_cache_loc && k_pool && v_pool && table && seq_lens, TS_EINVAL,
             "ts_kv_store: NULL tensor argument");
  TS_REQUIRE(cfg->page_size == 1, TS_EINVAL, "ts_kv_store appends to a per-token table (page_size 1)");
  TS_REQUIRE(batch >= 1 && pool_rows >= 1 && max_tokens >= 1, TS_EINVAL,
             "ts_kv_store: batch=%d pool_rows=%lld max_tokens=%d out of range", batch,
             (long long)pool_rows, max_tokens);
  TS_REQUIRE(batch == 1 || table_stride >= max_tokens, TS_EINVAL,
             "ts_kv_store: table_stride %lld < max_tokens %d", (long long)table_stride, max_tokens);
  const int row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  hipLaunchKernelGGL(kv_store_kernel, dim3((unsigned)batch), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)k, (const uint4*)v, out_cache_loc, (uint4*)k_pool, (uint4*)v_pool,
                     pool_rows, table, table_stride, seq_lens, row_vec, max_tokens);
  return check_launch("kv_store_kernel");
}

extern "C" int ts_kv_store_chunk(const ts_config* cfg, const void* k, const void* v,
                                 const int32_t* out_cache_loc, int32_t rows, void* k_pool,
                                 void* v_pool, int64_t pool_rows, int32_t* table, int32_t* seq_len,
                                 int32_t max_tokens, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(k && v && out_cache_loc && k_pool && v_pool && table && seq_len, TS_EINVAL,
             "ts_kv_store_chunk: NULL tensor argument");
  TS_REQUIRE(cfg->page_size == 1, TS_EINVAL,
             "ts_kv_store_chunk appends to a per-token table (page_size 1)");
  TS_REQUIRE(rows >= 0 && pool_rows >= 1 && max_tokens >= 1, TS_EINVAL,
             "ts_kv_store_chunk: rows=%d pool_rows=%lld max_tokens=%d out of range", rows,
             (long long)pool_rows, max_tokens);
  if (rows == 0) return TS_OK;
  const int row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  hipLaunchKernelGGL(kv_store_chunk_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream,
                     (const uint4*)k, (const uint4*)v, out_cache_loc, (uint4*)k_pool, (uint4*)v_pool,
                     pool_rows, table, seq_len, row_vec, max_tokens);
  TS_TRY(check_launch("kv_store_chunk_kernel"));
  hipLaunchKernelGGL(seq_len_add_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, seq_len, rows,
                     max_tokens);
  return check_launch("seq_len_add_kernel");
}
