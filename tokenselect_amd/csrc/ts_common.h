// Shared host/device helpers for libtokenselect_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tokenselect.h"

namespace ts {

// ---------------------------------------------------------------- host side
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
int validate_config(const ts_config* cfg);
int validate_batch(const ts_config* cfg, const ts_batch* bt);
bool group_supported(int num_kv_heads, int group);

#define TS_REQUIRE(cond, code, ...)                     \
  do {                                                  \
    if (!(cond)) return ::ts::fail((code), __VA_ARGS__); \
  } while (0)

#define TS_TRY(expr)            \
  do {                          \
    int _rc = (expr);           \
    if (_rc != TS_OK) return _rc; \
  } while (0)

// Device buffers are read and written with 16-byte vector accesses and 8-byte atomics:
// what hipMalloc and the framework allocators return is aligned far beyond that, a view
// at an odd offset is not, and would fault the device instead of failing a call.
#define TS_REQUIRE_ALIGNED(ptr, bytes, what)                                                   \
  TS_REQUIRE((reinterpret_cast<uintptr_t>(ptr) & ((bytes)-1)) == 0, TS_EINVAL,                  \
             "%s must be aligned to %d bytes", what, (int)(bytes))

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Candidate rows per workgroup of the scoring pass, shared by the launcher,
// the statistics merge and the workspace query.
int score_tokens_per_block(int64_t total_candidates, int num_heads);

// Words the rotation kernel clears on the side: `count` pieces of `words` 32-bit
// words, `stride` words apart (all zero: nothing to clear).
struct ZeroRegion {
  uint32_t* base = nullptr;
  int64_t stride = 0;
  int words = 0;
  int count = 0;
};
// What one such launch clears: up to four regions.
constexpr int kZeroRegions = 4;
struct ZeroSet {
  ZeroRegion r[kZeroRegions];
  int used = 0;
  bool overflow = false;  // a region did not fit: the launchers refuse such a set
  void add(const ZeroRegion& region) {
    if (region.count <= 0 || region.words <= 0) return;
    if (used < kZeroRegions)
      r[used++] = region;
    else
      overflow = true;
  }
  int64_t total() const {
    int64_t t = 0;
    for (int i = 0; i < used; ++i) t += (int64_t)r[i].count * r[i].words;
    return t;
  }
};
// Thread `gid` of `threads` clears its share of every region.
__device__ __forceinline__ void clear_regions(const ZeroSet& zero, int64_t gid, int64_t threads) {
#pragma unroll
  for (int i = 0; i < kZeroRegions; ++i) {
    if (i >= zero.used) break;
    const ZeroRegion& z = zero.r[i];
    for (int64_t w = gid; w < (int64_t)z.count * z.words; w += threads)
      z.base[(w / z.words) * z.stride + w % z.words] = 0u;
  }
}
// Chunk fingerprint (ts_prefill.hip) with the same side job as launch_rope: the
// regions are cleared by the same launch.
// The K/V rows of a prefill chunk, stored by the fingerprint launch on the side (as
// kv_store_chunk_kernel stores them): slots chosen by the caller, one per row.
struct ChunkStore {
  const uint4* k;  // [rows, Hkv*D] bf16 as 16-byte pieces
  const uint4* v;
  const int32_t* loc;
  uint4* k_pool;
  uint4* v_pool;
  int64_t pool_rows;
  int32_t* table;    // the request's row
  int32_t* seq_len;  // the request's length word
  int rows, row_vec, max_tokens;
  int workgroups;    // of the launch that store (set by the launcher)
};
int launch_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                       const float* sin_table, int64_t table_rows, void* qf, const ZeroSet& zero,
                       hipStream_t stream, const ChunkStore* store = nullptr);
int launch_rope(const void* x, void* out, const float* cos_table, const float* sin_table,
                const int64_t* position_ids, int64_t table_rows, int64_t rows, int heads, int dim,
                const ZeroSet& zero, hipStream_t stream);

// Selection-cache decision (ts_selcache.hip); gave_up_len: see ts_batch.rerun (NULL: an
// ordinary step).
int launch_selcache(const ts_config* cfg, const ts_batch* bt, const void* qf, const ts_selcache* cache,
                    int32_t* hit, const int32_t* gave_up_len, hipStream_t stream);

// The fingerprint rotation of a decode step (one query row per request, q_cos / q_sin the
// [D] table rows of its position) and the cache decision in one launch, which also clears
// the regions of `zero`.
// The new token's K/V rows of a decode step, stored by the first launch of the layer (as
// kv_store_kernel stores them): slots chosen by the caller, one per request.
struct StepStore {
  const uint4* k;  // [B, Hkv*D] bf16 as 16-byte pieces
  const uint4* v;
  const int32_t* loc;
  uint4* k_pool;
  uint4* v_pool;
  int64_t pool_rows;
  int32_t* table;
  int64_t table_stride;
  int32_t* seq_lens;
  int row_vec;     // 16-byte pieces per row
  int max_tokens;
  // With a page pool (free_pages != NULL; loc is not read): the slots come from the table and
  // the pool as kv_store_paged_kernel takes them.
  const int32_t* free_pages;
  int32_t* free_count;
  uint32_t* ticket;
  int page_shift;
};
int launch_rope_selcache(const ts_config* cfg, const ts_batch* bt, const void* q, void* qf,
                         const float* q_cos, const float* q_sin, const ts_selcache* cache, int32_t* hit,
                         const int32_t* gave_up_len, const ZeroSet& zero, hipStream_t stream,
                         const StepStore* store = nullptr);

// Sparse decode attention (ts_attn.hip).  The kernel counts its workgroups in per
// (request, KV head) tickets inside the workspace, which must be zero at launch:
// tickets_clear = false makes the launcher clear them first, true says an earlier
// kernel of the stream already did (attn_tickets() tells it where they are).
uint32_t* attn_tickets(const ts_config* cfg, int batch, int max_sel_len, void* workspace);
// Tickets per request (the words to clear): one per KV head.
int attn_tickets_per_request(const ts_config* cfg);
// clear_after: regions that the kernel clears on the side (the counters of the stream's
// next selection), or NULL.
int launch_attn(const ts_config* cfg, const void* q, const void* k_pool, const void* v_pool,
                int64_t pool_rows, const int32_t* sel, int64_t sel_stride, const int32_t* sel_len,
                int batch, int max_sel_len, void* out, void* workspace, bool tickets_clear,
                hipStream_t stream, const ZeroSet* clear_after = nullptr);

constexpr int kHeadDim = 128;
constexpr float kNegBig = -3.0e38f;  // finite stand-in for -inf in running maxima

// -------------------------------------------------------------- device side
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }

// Round-to-nearest-even, NaN kept quiet: the rounding torch applies on .to(bfloat16).
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// Two floats to packed bf16, round to nearest even, in one v_cvt_pk_bf16_f32.
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
constexpr int kRowRor1 = 0x121, kRowRor2 = 0x122, kRowRor4 = 0x124, kRowRor8 = 0x128;

// Sum over the 16 lanes of a DPP row; every lane of the row gets the total.
__device__ __forceinline__ float row16_sum(float x) {
  x += dpp_move<kRowRor8>(x);
  x += dpp_move<kRowRor4>(x);
  x += dpp_move<kRowRor2>(x);
  x += dpp_move<kRowRor1>(x);
  return x;
}

// sin and cos of an angle of up to some 1e5 radians: two-constant reduction by
// 2 pi (hi + lo parts, each product exact inside the FMA), then the hardware
// functions on [-pi, pi].
__device__ __forceinline__ void sincos_reduced(float x, float& sn, float& cs) {
  const float k = rintf(x * 0.15915494309189535f);
  float r = fmaf(-k, 6.2831854820251465f, x);
  r = fmaf(-k, -1.7484555e-07f, r);
  sn = __sinf(r);
  cs = __cosf(r);
}

// One element of the scoring query's rotation (RotaryEmbedding.apply_rotary_pos_emb,
// tr.py:98-107): own * cos + (+-other) * sin, where `other` is the element 64 dims away and
// enters negated for the lower half.  Products and the sum are rounded one by one (no FMA
// contraction), which is what the reference's elementwise torch expression does.
__device__ __forceinline__ float rotate_element(float own, float other, float cs, float sn, bool lower) {
#pragma clang fp contract(off)
  const float a = own * cs;
  const float b = (lower ? -other : other) * sn;
  return a + b;
}

// Merge two (max, sum-of-exp) softmax partials.
__device__ __forceinline__ void softmax_merge(float& m, float& l, float m2, float l2) {
  float mm = fmaxf(m, m2);
  l = l * __expf(m - mm) + l2 * __expf(m2 - mm);
  m = mm;
}

__device__ __forceinline__ void row16_softmax_merge(float& m, float& l) {
  softmax_merge(m, l, dpp_move<kRowRor8>(m), dpp_move<kRowRor8>(l));
  softmax_merge(m, l, dpp_move<kRowRor4>(m), dpp_move<kRowRor4>(l));
  softmax_merge(m, l, dpp_move<kRowRor2>(m), dpp_move<kRowRor2>(l));
  softmax_merge(m, l, dpp_move<kRowRor1>(m), dpp_move<kRowRor1>(l));
}

// Per-request geometry of the selection, evaluated on the device so that no
// host synchronisation is needed (tr.py:376-378, 424-426).
struct ReqGeom {
  int seq_len;  // L
  int k;        // per-request top-k
  int n;        // candidates = L - n_init - n_local (0 when dense)
  bool dense;   // n_init + k + n_local >= L
};

// seq_lens[b] is clamped to the host's max_seq_len, the bound every buffer and
// grid was sized for.
__device__ __forceinline__ ReqGeom request_geometry(const int32_t* seq_lens, const int32_t* k_per_req,
                                                    int b, int n_init, int n_local, int top_k,
                                                    int max_seq_len) {
  ReqGeom g;
  g.seq_len = min(max(seq_lens[b], 0), max_seq_len);
  int k = k_per_req ? k_per_req[b] : top_k;
  g.k = k < 0 ? 0 : (k > top_k ? top_k : k);
  g.dense = (n_init + g.k + n_local >= g.seq_len);
  g.n = g.dense ? 0 : g.seq_len - n_init - n_local;
  return g;
}

// Logical position -> physical KV slot through the (paged) table; page sizes are
// powers of two.  The slot is clamped to the pool so that a corrupt table cannot
// fault the GPU.
__device__ __forceinline__ uint32_t lookup_slot(const int32_t* tab, int pos, int page_size,
                                                int page_shift, uint32_t pool_rows) {
  const uint32_t slot =
      ((uint32_t)tab[pos >> page_shift] << page_shift) + (uint32_t)(pos & (page_size - 1));
  return slot < pool_rows ? slot : pool_rows - 1;
}

static inline int page_shift_of(int page_size) {
  if (page_size <= 0 || (page_size & (page_size - 1))) return -1;
  int s = 0;
  while ((1 << s) < page_size) ++s;
  return s;
}

}  // namespace ts
