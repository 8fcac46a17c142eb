// Criticality scoring: scores[h,t] = q[h,:] . K[slot(t), kv(h), :] streamed over the
// paged KV cache (the reference's paged_matmul_kernel, tr.py:166-231), plus the
// per-head softmax statistics the soft vote needs (tr.py:361).
//
// The pass is bound by HBM: every candidate row (Hkv*256 bytes) is read exactly
// once for all H query heads.  The dot products go through the matrix cores, not
// because the shape is a dense GEMM (it is 4 to 8 query rows per KV head) but
// because one v_mfma_f32_16x16x32_bf16 replaces 64 dot/reduce/select vector
// instructions and leaves the wavefront free to keep loads in flight:
//
//   B operand = keys:    lane l holds token (l%16) of a 16-token tile, 8 dims
//                        [32c + 8(l/16), +8) of one KV head - a 128-bit load
//                        straight from HBM into the operand registers;
//   A operand = queries: row 4*(g%4) + g/4 holds query g of the KV head, so
//   D result:            lane l, register r = score of query (l/16) + 4r for
//                        token l%16 - already one token per lane, 16
//                        consecutive tokens per 16-lane row: a 64-byte store
//                        per head, no cross-lane traffic at all.
//
// Products of bf16 pairs are exact in fp32 and the accumulation is fp32.
// Loads are double-buffered in half iterations (16 x 128-bit loads per lane
// each) and the table entry of the next tile is fetched one iteration ahead.
#include "ts_common.h"

namespace ts {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct ScoreArgs {
  const uint16_t* qf;      // [B,H,128] bf16 rotated fingerprints
  const uint16_t* k_pool;  // [pool_rows,Hkv,128] bf16
  uint32_t pool_rows;
  const int32_t* seq_lens;
  const int32_t* table;
  int64_t table_stride;
  const int32_t* k_per_req;
  const int32_t* skip;
  int n_init, n_local, top_k, page_size, page_shift, max_seq_len;
  int64_t direct_n;  // >= 0: paged_matmul mode, candidates are table[0..direct_n)
  void* scores;
  int64_t score_stride;  // elements between head rows
  float* partials;       // [B,H,nchunks,2] or NULL
  int nchunks;
  int tokens_per_block;
  int num_heads;
  int head_map;
};

template <int HKV, int G>
__device__ __forceinline__ int head_of(int kvh, int g, int head_map) {
  return head_map == TS_HEADMAP_MOD ? kvh + HKV * g : kvh * G + g;
}

// One iteration of a wave covers TG tiles of 16 tokens and all HKV heads: always
// 8 (tile, KV head) units = 32 loads of 1 KB.  Units 0-3 and 4-7 alternate
// between two register buffers.
template <int HKV, int G, bool OUT_BF16>
__global__ __launch_bounds__(256, 1) void score_kernel(ScoreArgs a) {
  constexpr int TG = 8 / HKV;
  constexpr int UNITS = 8;
  constexpr int HALF = UNITS / 2;
  constexpr int NR = (G + 3) / 4;  // result registers in use per unit
  constexpr int ITER = 16 * TG;    // tokens per iteration
  constexpr uint32_t ROW_BYTES = HKV * kHeadDim * 2;

  const int b = blockIdx.y;
  int n, first_pos;
  if (a.direct_n >= 0) {
    n = (int)a.direct_n;
    first_pos = 0;
  } else {
    if (a.skip && a.skip[b]) return;
    ReqGeom geo = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k,
                                   a.max_seq_len);
    n = geo.n;
    first_pos = a.n_init;
  }
  const int block_lo = blockIdx.x * a.tokens_per_block;
  if (block_lo >= n) return;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rg = lane >> 4;   // k-group of the operands, row group of the result
  const int col = lane & 15;  // token inside a tile
  const int H = a.num_heads;
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;

  // A operands: query (col/4 + 4*(col%4)) of each KV head, dims [32c + 8rg, +8).
  bf16x8_t qa[HKV][4];
  {
    const int g = (col >> 2) + 4 * (col & 3);
#pragma unroll
    for (int kvh = 0; kvh < HKV; ++kvh) {
      const int h = head_of<HKV, G>(kvh, g < G ? g : 0, a.head_map);
      const uint16_t* qrow = a.qf + ((size_t)b * H + h) * kHeadDim + rg * 8;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (g < G) v = *(const uint4*)(qrow + c * 32);
        qa[kvh][c] = __builtin_bit_cast(bf16x8_t, v);
      }
    }
  }

  float run_m[HKV][NR], run_l[HKV][NR];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      run_m[kvh][r] = kNegBig;
      run_l[kvh][r] = 0.f;
    }

  const int per_wave = a.tokens_per_block >> 2;
  const int wave_lo = block_lo + wave * per_wave;
  const int wave_hi = min(wave_lo + per_wave, n);

  // Lane (rg, col) addresses token `tile + col` of every tile.  The table load and
  // the slot arithmetic are split so that the entry of the next iteration is
  // requested a whole iteration before it is needed.  Positions past the wave's
  // range are clamped to its last token: every load stays in bounds and no branch
  // splits the load pipeline.
  const int last_pos = first_pos + max(wave_hi - 1, 0);
  const int page_mask = a.page_size - 1;
  auto table_entry = [&](int tile) -> int32_t {
    const int pos = min(first_pos + tile + col, last_pos);
    return tab[pos >> a.page_shift];
  };
  auto row_ptr = [&](int32_t entry, int tile) -> const char* {
    const int pos = min(first_pos + tile + col, last_pos);
    uint32_t slot = ((uint32_t)entry << a.page_shift) + (uint32_t)(pos & page_mask);
    slot = slot < a.pool_rows ? slot : a.pool_rows - 1;
    return (const char*)a.k_pool + (size_t)slot * ROW_BYTES + rg * 16;
  };

  uint4 buf0[HALF][4], buf1[HALF][4];
  auto issue = [&](uint4 (&buf)[HALF][4], auto& rows, int first_unit) {
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
      const int u = first_unit + i;
      const char* p = rows[u / HKV] + (u % HKV) * (kHeadDim * 2);
#pragma unroll
      for (int c = 0; c < 4; ++c) buf[i][c] = *(const uint4*)(p + c * 64);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto multiply = [&](const uint4 (&buf)[HALF][4], f32x4_t (&acc)[UNITS], int first_unit) {
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
      const int u = first_unit + i;
      f32x4_t d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; ++c)
        d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[u % HKV][c],
                                                    __builtin_bit_cast(bf16x8_t, buf[i][c]), d, 0, 0, 0);
      acc[u] = d;
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  const char* rows_cur[TG];
  const char* rows_next[TG];
  if (wave_lo < wave_hi) {
#pragma unroll
    for (int t = 0; t < TG; ++t) rows_cur[t] = row_ptr(table_entry(wave_lo + 16 * t), wave_lo + 16 * t);
    issue(buf0, rows_cur, 0);
  }

  for (int base = wave_lo; base < wave_hi; base += ITER) {
    int32_t entry_next[TG];
#pragma unroll
    for (int t = 0; t < TG; ++t) entry_next[t] = table_entry(base + ITER + 16 * t);
    __builtin_amdgcn_sched_barrier(0);

    f32x4_t acc[UNITS];
    issue(buf1, rows_cur, HALF);
    multiply(buf0, acc, 0);
#pragma unroll
    for (int t = 0; t < TG; ++t) rows_next[t] = row_ptr(entry_next[t], base + ITER + 16 * t);
    issue(buf0, rows_next, 0);
    multiply(buf1, acc, HALF);
#pragma unroll
    for (int t = 0; t < TG; ++t) rows_cur[t] = rows_next[t];

    // Lane (rg, col), register r of unit (tile t, head kvh): query rg + 4r, token
    // base + 16t + col.
#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      const int t = u / HKV, kvh = u % HKV;
      const int tok = base + 16 * t + col;
#pragma unroll
      for (int r = 0; r < NR; ++r) {
        const int g = rg + 4 * r;
        if (g < G && tok < wave_hi) {
          const int h = head_of<HKV, G>(kvh, g, a.head_map);
          const float x = acc[u][r];
          const size_t at = ((size_t)b * H + h) * (size_t)a.score_stride + (size_t)tok;
#ifndef TS_DBG_NOSTORE
          if (OUT_BF16)
            ((uint16_t*)a.scores)[at] = f32_to_bf16(x);
          else
            ((float*)a.scores)[at] = x;
#else
          if (x == 1234.5678f) ((float*)a.scores)[at] = x;
#endif
#ifdef TS_DBG_NOSTATS
          run_l[kvh][r] += x;
          continue;
#endif
          // Online (max, sum exp) with a single exponential per element.
          const float d = x - run_m[kvh][r];
          const float e = __expf(-fabsf(d));
          if (d > 0.f) {
            run_l[kvh][r] = run_l[kvh][r] * e + 1.f;
            run_m[kvh][r] = x;
          } else {
            run_l[kvh][r] += e;
          }
        }
      }
    }
  }

  if (a.partials == nullptr) return;

  __shared__ float sm_m[4][4][HKV][NR];
  __shared__ float sm_l[4][4][HKV][NR];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      float m = run_m[kvh][r], l = run_l[kvh][r];
      row16_softmax_merge(m, l);
      if (col == 0) {
        sm_m[wave][rg][kvh][r] = m;
        sm_l[wave][rg][kvh][r] = l;
      }
    }
  __syncthreads();
  if ((int)threadIdx.x < H) {
    const int h = threadIdx.x;
    float m = kNegBig, l = 0.f;
    for (int w = 0; w < 4; ++w)
      for (int g4 = 0; g4 < 4; ++g4)
        for (int kvh = 0; kvh < HKV; ++kvh)
          for (int r = 0; r < NR; ++r) {
            const int g = g4 + 4 * r;
            if (g < G && head_of<HKV, G>(kvh, g, a.head_map) == h)
              softmax_merge(m, l, sm_m[w][g4][kvh][r], sm_l[w][g4][kvh][r]);
          }
    float* p = a.partials + (((size_t)b * H + h) * a.nchunks + blockIdx.x) * 2;
    p[0] = m;
    p[1] = l;
  }
}

template <bool OUT_BF16>
static int launch_score(int hkv, int group, const ScoreArgs& a, dim3 grid, hipStream_t stream) {
#define TS_SCORE_CASE(HKV_, G_)                                                              \
  if (hkv == HKV_ && group == G_) {                                                          \
    hipLaunchKernelGGL((score_kernel<HKV_, G_, OUT_BF16>), grid, dim3(256), 0, stream, a);   \
    return check_launch("score_kernel");                                                     \
  }
#define TS_SCORE_ROW(HKV_) \
  TS_SCORE_CASE(HKV_, 1) TS_SCORE_CASE(HKV_, 2) TS_SCORE_CASE(HKV_, 4) TS_SCORE_CASE(HKV_, 7) TS_SCORE_CASE(HKV_, 8)
  TS_SCORE_ROW(1)
  TS_SCORE_ROW(2)
  TS_SCORE_ROW(4)
  TS_SCORE_ROW(8)
#undef TS_SCORE_ROW
#undef TS_SCORE_CASE
  return fail(TS_ESHAPE, "unsupported head shape: num_kv_heads=%d group=%d", hkv, group);
}

}  // namespace ts

using namespace ts;

extern "C" {

size_t ts_score_partials_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  const int tpb = score_tokens_per_block((int64_t)batch * max_seq_len);
  const size_t nchunks = (size_t)ceil_div(max_seq_len, tpb);
  return align_up((size_t)batch * cfg->num_heads * nchunks * 2 * sizeof(float), 256);
}

int ts_score(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
             int64_t pool_rows, const int32_t* skip, float* scores, int64_t score_stride,
             float* partials, size_t partials_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(qf && k_pool && scores && partials, TS_EINVAL, "ts_score: NULL tensor argument");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(score_stride >= max_n && score_stride >= 1, TS_EWORKSPACE,
             "score_stride %lld < max candidates %d", (long long)score_stride, max_n);
  const size_t need = ts_score_partials_bytes(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(partials_bytes >= need, TS_EWORKSPACE, "ts_score: partials %zu bytes < required %zu",
             partials_bytes, need);
  if (max_n <= 0) return TS_OK;  // every request is dense

  ScoreArgs a;
  a.qf = (const uint16_t*)qf;
  a.k_pool = (const uint16_t*)k_pool;
  a.pool_rows = (uint32_t)pool_rows;
  a.seq_lens = bt->seq_lens;
  a.table = bt->table;
  a.table_stride = bt->table_stride;
  a.k_per_req = bt->k_per_req;
  a.skip = skip;
  a.n_init = cfg->n_init;
  a.n_local = cfg->n_local;
  a.top_k = cfg->top_k;
  a.max_seq_len = bt->max_seq_len;
  a.page_size = cfg->page_size;
  a.page_shift = page_shift_of(cfg->page_size);
  a.direct_n = -1;
  a.scores = scores;
  a.score_stride = score_stride;
  a.partials = partials;
  a.tokens_per_block = score_tokens_per_block((int64_t)bt->batch * bt->max_seq_len);
  a.nchunks = (int)ceil_div(bt->max_seq_len, a.tokens_per_block);
  a.num_heads = cfg->num_heads;
  a.head_map = cfg->head_map;
  const dim3 grid((unsigned)ceil_div(max_n, a.tokens_per_block), (unsigned)bt->batch);
  return launch_score<false>(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads, a, grid,
                             (hipStream_t)stream);
}

int ts_paged_matmul(const void* query, const void* token, int64_t pool_rows,
                    const int32_t* indices, void* scores, int32_t scores_dtype, int64_t n,
                    int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                    ts_stream_t stream) {
  TS_REQUIRE(query && token && indices && scores, TS_EINVAL, "ts_paged_matmul: NULL tensor argument");
  TS_REQUIRE(head_dim == kHeadDim, TS_ESHAPE, "head_dim %d not supported (only 128)", head_dim);
  TS_REQUIRE(num_heads > 0 && num_kv_heads > 0 && num_heads % num_kv_heads == 0, TS_ESHAPE,
             "num_heads %d / num_kv_heads %d invalid", num_heads, num_kv_heads);
  TS_REQUIRE(group_supported(num_kv_heads, num_heads / num_kv_heads), TS_ESHAPE,
             "unsupported head shape: num_kv_heads=%d group=%d", num_kv_heads,
             num_heads / num_kv_heads);
  TS_REQUIRE(scores_dtype == TS_DTYPE_F32 || scores_dtype == TS_DTYPE_BF16, TS_EINVAL,
             "scores_dtype %d unknown", scores_dtype);
  TS_REQUIRE(n >= 0 && n <= 0x7fffffffLL, TS_EINVAL, "n %lld out of range", (long long)n);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  if (n == 0) return TS_OK;

  ScoreArgs a;
  a.qf = (const uint16_t*)query;
  a.k_pool = (const uint16_t*)token;
  a.pool_rows = (uint32_t)pool_rows;
  a.seq_lens = nullptr;
  a.table = indices;
  a.table_stride = 0;
  a.k_per_req = nullptr;
  a.skip = nullptr;
  a.n_init = a.n_local = 0;
  a.top_k = 1;
  a.max_seq_len = 0;
  a.page_size = 1;
  a.page_shift = 0;
  a.direct_n = n;
  a.scores = scores;
  a.score_stride = n;
  a.partials = nullptr;
  a.tokens_per_block = score_tokens_per_block(n);
  a.nchunks = (int)ceil_div(n, a.tokens_per_block);
  a.num_heads = num_heads;
  a.head_map = TS_HEADMAP_MOD;
  const dim3 grid((unsigned)a.nchunks, 1);
  if (scores_dtype == TS_DTYPE_BF16)
    return launch_score<true>(num_kv_heads, num_heads / num_kv_heads, a, grid, (hipStream_t)stream);
  return launch_score<false>(num_kv_heads, num_heads / num_kv_heads, a, grid, (hipStream_t)stream);
}

}  // extern "C"
