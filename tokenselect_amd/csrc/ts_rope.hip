// Rotation of the scoring query: RotaryEmbedding.apply_rotary_pos_emb, tr.py:98-107.
#include <algorithm>

#include "ts_common.h"

namespace ts {

// One thread per (row, head, i < dim/2): writes out[i] and out[i + dim/2].
// Products and the sum are rounded one by one (no FMA contraction), which is
// what the reference's elementwise torch expression does, so that the result is
// bit-identical for identical tables.
__global__ __launch_bounds__(256) void rope_apply_kernel(const uint16_t* __restrict__ x,
                                                         uint16_t* __restrict__ out,
                                                         const float* __restrict__ cos_table,
                                                         const float* __restrict__ sin_table,
                                                         const int64_t* __restrict__ position_ids,
                                                         int64_t table_rows, int64_t rows, int heads,
                                                         int dim, ZeroSet zero) {
#pragma clang fp contract(off)
  const int half = dim >> 1;
  const int64_t pairs = rows * heads * half;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  // Counters the later kernels of a decode step accumulate into.
  clear_regions(zero, gid, (int64_t)gridDim.x * blockDim.x);
  if (gid >= pairs) return;
  const int i = (int)(gid % half);
  const int64_t rh = gid / half;
  const int64_t row = rh / heads;
  int64_t pos = position_ids ? position_ids[row] : 0;
  if (pos < 0) pos = 0;
  if (pos >= table_rows) pos = table_rows - 1;
  const float* c = cos_table + pos * dim;
  const float* s = sin_table + pos * dim;
  const int64_t base = rh * dim;
  const float x1 = bf16_to_f32(x[base + i]);
  const float x2 = bf16_to_f32(x[base + i + half]);
  const float lo = rotate_element(x1, x2, c[i], s[i], true);
  const float hi = rotate_element(x2, x1, c[i + half], s[i + half], false);
  out[base + i] = f32_to_bf16(lo);
  out[base + i + half] = f32_to_bf16(hi);
}

int launch_rope(const void* x, void* out, const float* cos_table, const float* sin_table,
                const int64_t* position_ids, int64_t table_rows, int64_t rows, int heads, int dim,
                const ZeroSet& zero, hipStream_t stream) {
  TS_REQUIRE(!zero.overflow, TS_EINVAL, "internal: more than %d regions to clear in one launch", kZeroRegions);
  const int64_t pairs = rows * heads * (dim / 2);
  // Enough workgroups for the clearing on the side as well: four words per thread.
  const int64_t to_clear = zero.total();
  const int64_t blocks = std::max(ceil_div(pairs, 256), ceil_div(to_clear, 1024));
  TS_REQUIRE(blocks <= 0x7fffffff, TS_EINVAL, "ts_rope_apply: too many rows");
  hipLaunchKernelGGL(rope_apply_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                     (const uint16_t*)x, (uint16_t*)out, cos_table, sin_table, position_ids,
                     table_rows, rows, heads, dim, zero);
  return check_launch("rope_apply_kernel");
}

}  // namespace ts

using namespace ts;

extern "C" int ts_rope_apply(const void* x, void* out, const float* cos_table,
                             const float* sin_table, const int64_t* position_ids,
                             int64_t table_rows, int64_t rows, int32_t heads, int32_t dim,
                             ts_stream_t stream) {
  TS_REQUIRE(x && out && cos_table && sin_table, TS_EINVAL, "ts_rope_apply: NULL tensor argument");
  TS_REQUIRE(rows >= 0 && heads >= 1 && table_rows >= 1, TS_EINVAL,
             "ts_rope_apply: rows=%lld heads=%d table_rows=%lld out of range", (long long)rows, heads,
             (long long)table_rows);
  TS_REQUIRE(dim >= 2 && dim % 2 == 0, TS_ESHAPE, "ts_rope_apply: dim %d must be even", dim);
  if (rows == 0) return TS_OK;
  return launch_rope(x, out, cos_table, sin_table, position_ids, table_rows, rows, heads, dim,
                     ZeroSet{}, (hipStream_t)stream);
}
