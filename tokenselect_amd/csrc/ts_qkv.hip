// QKV projection of a decode step with the KV store as its epilogue: the step
// before the hot path.  The serving stack computes qkv = x W^T in the model
// (LlamaAttention.forward) and the patched attention then scatters K and V into the
// pool and appends the slot to the token table (patched_radix_attention_store_kv_cache
// tr.py:844-854, add_k_cache tr.py:332-336); here the projection writes the K and V
// rows straight to their pool slot, so the [B, Hkv*D] staging rows, their copies
// and the separate store launch disappear.
//
// With a handful of rows in x the product is a stream over W (bound: HBM).  A
// wavefront owns two or three whole rows of W: a lane reads up to eight 16-byte pieces
// of each (all requested before the first is used, before x is staged), multiplies
// them with the matching pieces of x from LDS (bf16, staged once per workgroup of
// eight wavefronts) and the wavefront reduces its sums (rows x B) on its own: no
// exchange between wavefronts.
#include "ts_pages.h"

namespace ts {

constexpr int kQkvMaxBatch = 8;      // rows of x
constexpr int kQkvWaves = 8;         // wavefronts per workgroup
constexpr int kQkvPieces = 8;        // 16-byte pieces of a row per lane
constexpr int kQkvMaxHidden = 4096;  // 64 lanes x kQkvPieces x 8 elements

struct QkvArgs {
  const uint16_t* x;     // [B, hidden] bf16
  const uint16_t* w;     // [n_out, hidden] bf16
  const uint16_t* bias;  // [n_out] bf16 or NULL
  int hidden, n_out, q_cols, kv_cols;
  const int32_t* loc;    // [B] pool slot of the new token
  uint16_t* q_out;       // [B, q_cols]
  uint16_t* k_pool;
  uint16_t* v_pool;
  int64_t pool_rows;
  int32_t* table;
  int64_t table_stride;
  int32_t* seq_lens;
  int max_tokens;
  PagePool pool;  // free_pages != NULL: slots come from the table / the free list (ts_pages.h)
  int page_shift;
};

// a.lo * b.lo + a.hi * b.hi + c on packed bf16 pairs.
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c,
                                         false);
}

// W is read once: a non-temporal load keeps it from displacing the rest of the cache.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
__device__ __forceinline__ uint4 load_streaming(const uint4* p) {
  const u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// kQkvRows: rows of W per wavefront (two or three, whichever spreads the rows more evenly
// over the CUs).
template <int B, int kQkvRows>
__global__ __launch_bounds__(64 * kQkvWaves) void qkv_store_kernel(QkvArgs a) {
  extern __shared__ uint4 lds_x[];  // [B][hidden / 8]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kvec = a.hidden >> 3;  // 16-byte pieces per row
  const int n0 = (blockIdx.x * kQkvWaves + wave) * kQkvRows;

  // The wavefront's rows first: they do not depend on the copy of x.
  uint4 wv[kQkvRows][kQkvPieces];
#pragma unroll
  for (int r = 0; r < kQkvRows; ++r) {
    const uint4* row = (const uint4*)(a.w + (size_t)min(n0 + r, a.n_out - 1) * a.hidden);
#pragma unroll
    for (int j = 0; j < kQkvPieces; ++j) {
      const int v = lane + 64 * j;
      wv[r][j] = v < kvec ? load_streaming(row + v) : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  for (int i = tid; i < B * kvec; i += 64 * kQkvWaves) lds_x[i] = ((const uint4*)a.x)[i];
  __syncthreads();

  float acc[kQkvRows][B];
#pragma unroll
  for (int r = 0; r < kQkvRows; ++r)
#pragma unroll
    for (int b = 0; b < B; ++b) acc[r][b] = 0.f;
  // Two bf16 products per instruction, accumulated in fp32 (v_dot2c_f32_bf16): the operands
  // stay packed as they were loaded, nothing is unpacked.
#pragma unroll
  for (int j = 0; j < kQkvPieces; ++j) {
    const int v = min(lane + 64 * j, kvec - 1);  // past the row: W piece is zero
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const uint4 xv = lds_x[b * kvec + v];
#pragma unroll
      for (int r = 0; r < kQkvRows; ++r) {
        acc[r][b] = dot2_bf16(wv[r][j].x, xv.x, acc[r][b]);
        acc[r][b] = dot2_bf16(wv[r][j].y, xv.y, acc[r][b]);
        acc[r][b] = dot2_bf16(wv[r][j].z, xv.z, acc[r][b]);
        acc[r][b] = dot2_bf16(wv[r][j].w, xv.w, acc[r][b]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < kQkvRows; ++r)
#pragma unroll
    for (int b = 0; b < B; ++b) {
      // (within a row of 16 lanes by DPP, the four rows through the LDS crossbar)
      acc[r][b] = row16_sum(acc[r][b]);
      acc[r][b] += __shfl_xor(acc[r][b], 16);
      acc[r][b] += __shfl_xor(acc[r][b], 32);
    }
  // Lane r * B + b writes y[b][n0 + r] (every lane holds every sum).
  float y = 0.f;
#pragma unroll
  for (int r = 0; r < kQkvRows; ++r)
#pragma unroll
    for (int b = 0; b < B; ++b)
      if (lane == r * B + b) y = acc[r][b];
  if (lane < kQkvRows * B) {
    const int r = lane / B, b = lane % B;
    const int n = n0 + r;
    if (n < a.n_out) {
      if (a.bias) y += bf16_to_f32(a.bias[n]);
      const uint16_t out = f32_to_bf16(y);
      if (n < a.q_cols) {
        a.q_out[(size_t)b * a.q_cols + n] = out;
      } else {
        int64_t slot = -1;
        if (a.pool.free_pages) {
          // The plan of request b, from the lengths as they were at launch: the
          // requests before it that take a page decide which page it takes.
          const int page_mask = (1 << a.page_shift) - 1;
          uint32_t rank = 0;
#pragma unroll
          for (int c = 0; c < B; ++c) {
            const int lc = a.seq_lens[c];
            rank += (c < b && lc >= 0 && lc < a.max_tokens && (lc & page_mask) == 0) ? 1u : 0u;
          }
          const int len = a.seq_lens[b];
          const bool room = len >= 0 && len < a.max_tokens;
          const AppendPlan plan = make_append_plan(
              a.table + (int64_t)b * a.table_stride, len, room, room && (len & page_mask) == 0, rank,
              max(*a.pool.free_count, 0), a.pool.free_pages, a.page_shift, page_mask,
              (uint32_t)a.pool_rows);
          if (plan.ok) slot = plan.slot;
        } else {
          slot = a.loc[b];
        }
        if (slot >= 0 && slot < a.pool_rows) {
          const int c = n - a.q_cols;
          if (c < a.kv_cols)
            a.k_pool[(size_t)slot * a.kv_cols + c] = out;
          else
            a.v_pool[(size_t)slot * a.kv_cols + (c - a.kv_cols)] = out;
        }
      }
    }
  }

  // Paged table: the launch's last workgroup commits the appends (nothing of the
  // snapshot the plans are made from changes before every workgroup is through).
  if (a.pool.free_pages) {
    __syncthreads();
    if (tid < 64)
      commit_appends(a.seq_lens, a.table, a.table_stride, B, a.pool, a.page_shift, a.max_tokens,
                     (uint32_t)a.pool_rows, lane, gridDim.x);
    return;
  }
  // Table append (add_k_cache tr.py:332-336) by the first workgroup; a full table
  // (tr.py:334 asserts) or a slot outside the pool leaves table and length alone.
  // (The K and V rows of a request whose table is full are still written to the
  // caller's slot: the other workgroups cannot consult a length that this one is
  // changing.  The reference asserts on the host before it appends, tr.py:334, and so
  // do the callers of this library.)
  if (blockIdx.x == 0 && tid < B) {
    const int b = tid;
    const int slot = a.loc[b];
    const int len = a.seq_lens[b];
    if (slot >= 0 && slot < a.pool_rows && len < a.max_tokens) {
      a.table[(int64_t)b * a.table_stride + len] = slot;
      a.seq_lens[b] = len + 1;
    }
  }
}

template <int B>
static int launch_qkv(const QkvArgs& a, hipStream_t stream) {
  const size_t lds = (size_t)B * a.hidden * 2;  // at most 64 KB
  // The kernel is one burst of loads per wavefront, and the slowest CU decides: 6144 rows
  // (Llama-3-8B) in 16-row workgroups are 384 workgroups, one and a half per CU, 16.3 us;
  // in 24-row workgroups 256, one per CU, 14.5 us; in 32-row workgroups 192: 16.8 us.
  static thread_local int cus_of[64] = {};  // by device, asked once per thread
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) {
    (void)hipGetLastError();
    device = 0;
  }
  int& cus = cus_of[device & 63];
  if (cus <= 0 &&
      (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)) {
    (void)hipGetLastError();
    cus = 256;
  }
  auto rounds = [&](int rows) { return ceil_div(ceil_div(a.n_out, rows * kQkvWaves), cus) * rows; };
  if (rounds(3) < rounds(2)) {
    hipLaunchKernelGGL((qkv_store_kernel<B, 3>), dim3((unsigned)ceil_div(a.n_out, 3 * kQkvWaves)),
                       dim3(64 * kQkvWaves), lds, stream, a);
  } else {
    hipLaunchKernelGGL((qkv_store_kernel<B, 2>), dim3((unsigned)ceil_div(a.n_out, 2 * kQkvWaves)),
                       dim3(64 * kQkvWaves), lds, stream, a);
  }
  return check_launch("qkv_store_kernel");
}

}  // namespace ts

using namespace ts;

extern "C" int ts_qkv_store(const ts_config* cfg, const void* x, const void* w, const void* bias,
                            int32_t hidden, const int32_t* out_cache_loc,
                            const ts_page_pool* pages, void* q_out,
                            void* k_pool, void* v_pool, int64_t pool_rows, int32_t* table,
                            int64_t table_stride, int32_t* seq_lens, int32_t batch,
                            int32_t max_tokens, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(x && w && q_out && k_pool && v_pool && table && seq_lens, TS_EINVAL,
             "ts_qkv_store: NULL tensor argument");
  TS_REQUIRE_ALIGNED(x, 16, "x");
  TS_REQUIRE_ALIGNED(w, 16, "w");
  TS_REQUIRE_ALIGNED(q_out, 16, "q_out");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  if (pages) {
    TS_REQUIRE(pages->free_pages && pages->free_count && pages->ticket, TS_EINVAL,
               "ts_qkv_store: page pool has a NULL array");
  } else {
    TS_REQUIRE(cfg->page_size == 1, TS_EINVAL,
               "ts_qkv_store: page_size %d needs a page pool", cfg->page_size);
    TS_REQUIRE(out_cache_loc != nullptr, TS_EINVAL, "ts_qkv_store: NULL out_cache_loc and no page pool");
  }
  TS_REQUIRE(batch >= 1 && batch <= kQkvMaxBatch, TS_ESHAPE,
             "ts_qkv_store: batch %d outside 1..%d (use a library GEMM and ts_kv_store)", batch,
             kQkvMaxBatch);
  TS_REQUIRE(hidden >= 8 && hidden % 8 == 0 && hidden <= kQkvMaxHidden, TS_ESHAPE,
             "ts_qkv_store: hidden %d must be a multiple of 8, at most %d", hidden, kQkvMaxHidden);
  TS_REQUIRE(pool_rows >= 1 && max_tokens >= 1, TS_EINVAL,
             "ts_qkv_store: pool_rows=%lld max_tokens=%d out of range", (long long)pool_rows,
             max_tokens);
  TS_REQUIRE(batch == 1 || table_stride * (int64_t)cfg->page_size >= max_tokens, TS_EINVAL,
             "ts_qkv_store: table_stride %lld x page_size %d < max_tokens %d", (long long)table_stride,
             cfg->page_size, max_tokens);
  QkvArgs a;
  a.pool = page_pool_of(pages);
  a.page_shift = page_shift_of(cfg->page_size);
  a.x = (const uint16_t*)x;
  a.w = (const uint16_t*)w;
  a.bias = (const uint16_t*)bias;
  a.hidden = hidden;
  a.q_cols = cfg->num_heads * cfg->head_dim;
  a.kv_cols = cfg->num_kv_heads * cfg->head_dim;
  a.n_out = a.q_cols + 2 * a.kv_cols;
  a.loc = out_cache_loc;
  a.q_out = (uint16_t*)q_out;
  a.k_pool = (uint16_t*)k_pool;
  a.v_pool = (uint16_t*)v_pool;
  a.pool_rows = pool_rows;
  a.table = table;
  a.table_stride = table_stride;
  a.seq_lens = seq_lens;
  a.max_tokens = max_tokens;
  switch (batch) {
    case 1: return launch_qkv<1>(a, (hipStream_t)stream);
    case 2: return launch_qkv<2>(a, (hipStream_t)stream);
    case 3: return launch_qkv<3>(a, (hipStream_t)stream);
    case 4: return launch_qkv<4>(a, (hipStream_t)stream);
    case 5: return launch_qkv<5>(a, (hipStream_t)stream);
    case 6: return launch_qkv<6>(a, (hipStream_t)stream);
    case 7: return launch_qkv<7>(a, (hipStream_t)stream);
    default: return launch_qkv<8>(a, (hipStream_t)stream);
  }
}
