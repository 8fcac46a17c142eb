// Criticality scoring: scores[h,t] = q[h,:] . K[slot(t), kv(h), :] streamed over the
// paged KV cache (the reference's paged_matmul_kernel, tr.py:166-231), plus the
// per-head softmax statistics the soft vote needs (tr.py:361).
//
// Data movement: a wavefront reads one token row (Hkv*256 bytes, contiguous in
// the pool) with 128-bit loads, 16 lanes per KV head, so every row is fetched
// from HBM exactly once for all H query heads.  The G = H/Hkv queries that share
// a KV head live in registers as packed bf16 pairs; products are exact and
// accumulated in fp32 (v_dot2_f32_bf16), then reduced over the 16 lanes of the
// DPP row.  Results of 16 consecutive rows are transposed into lanes so that the
// score store is one contiguous 64-byte segment per head.
#include "ts_common.h"

#ifndef TS_SCORE_SUBBATCH
#define TS_SCORE_SUBBATCH 4  // wave steps per load sub-batch: 4 or 8
#endif
#ifndef TS_SCORE_WAVES_PER_EU
#define TS_SCORE_WAVES_PER_EU 3
#endif

namespace ts {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

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

__device__ __forceinline__ float dot8(const uint4& k, const uint32_t (&q)[4]) {
  float acc = 0.f;
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, k.x),
                                        __builtin_bit_cast(bf16x2_t, q[0]), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, k.y),
                                        __builtin_bit_cast(bf16x2_t, q[1]), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, k.z),
                                        __builtin_bit_cast(bf16x2_t, q[2]), acc, false);
  acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, k.w),
                                        __builtin_bit_cast(bf16x2_t, q[3]), acc, false);
  return acc;
}

template <int HKV, int G>
__device__ __forceinline__ int head_of(int kvh, int g, int head_map) {
  return head_map == TS_HEADMAP_MOD ? kvh + HKV * g : kvh * G + g;
}

// Lane layout.  HKV >= 4: a wave step covers one token; 16-lane group `lg` reads
// KV heads lg, lg+4, ... (KVS 1-KB loads per row).  HKV < 4: a row is shorter
// than 1 KB, so a step covers TPW = 4/HKV tokens and group lg reads KV head
// lg % HKV of token lg / HKV.
template <int HKV, int G, bool OUT_BF16>
__global__ __launch_bounds__(256, ((HKV >= 4 ? HKV / 4 : 1) * G > 8 ? 2 : TS_SCORE_WAVES_PER_EU)) void score_kernel(ScoreArgs a) {
  constexpr int KVS = HKV >= 4 ? HKV / 4 : 1;
  constexpr int TPW = HKV >= 4 ? 1 : 4 / HKV;
  constexpr int TILE = 16 * TPW;

  const int b = blockIdx.y;
  int n, first_pos;
  if (a.direct_n >= 0) {
    n = (int)a.direct_n;
    first_pos = 0;
  } else {
    if (a.skip && a.skip[b]) return;
    ReqGeom geo = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
    n = geo.n;
    first_pos = a.n_init;
  }
  const int block_lo = blockIdx.x * a.tokens_per_block;
  if (block_lo >= n) return;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lg = lane >> 4, l16 = lane & 15;
  const int tok_sub = HKV >= 4 ? 0 : lg / HKV;
  const int H = a.num_heads;
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;

  uint32_t qreg[KVS][G][4];
  uint32_t kv_off[KVS];  // byte offset of this lane's 16 bytes inside a token row
#pragma unroll
  for (int s = 0; s < KVS; ++s) {
    const int kvh = HKV >= 4 ? lg + 4 * s : lg % HKV;
    kv_off[s] = (uint32_t)(kvh * kHeadDim + l16 * 8) * 2u;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int h = head_of<HKV, G>(kvh, g, a.head_map);
      const uint4 v = *(const uint4*)(a.qf + ((size_t)b * H + h) * kHeadDim + l16 * 8);
      qreg[s][g][0] = v.x;
      qreg[s][g][1] = v.y;
      qreg[s][g][2] = v.z;
      qreg[s][g][3] = v.w;
    }
  }

  float run_m[KVS][G], run_l[KVS][G];
#pragma unroll
  for (int s = 0; s < KVS; ++s)
#pragma unroll
    for (int g = 0; g < G; ++g) {
      run_m[s][g] = kNegBig;
      run_l[s][g] = 0.f;
    }

  const int per_wave = a.tokens_per_block >> 2;
  const int wave_lo = block_lo + wave * per_wave;
  const int wave_hi = min(wave_lo + per_wave, n);

  // A tile is 16 wave steps (16*TPW tokens) whose results are transposed into
  // the 16 lanes of a row.  It is loaded in sub-batches of SB steps that
  // alternate between two register buffers, so that the loads of the next
  // sub-batch are in flight while the current one is reduced.
  constexpr int SB = TS_SCORE_SUBBATCH;
  constexpr int NSB = 16 / SB;  // sub-batches per tile (even)
  uint4 buf0[SB][KVS], buf1[SB][KVS];

  // Lane i resolves the slot of token tile+i.  The table load and the slot
  // arithmetic are split so that the load of the next tile's entries is issued a
  // whole tile before its value is needed.  Out-of-range lanes and tiles are
  // clamped to the wave's last token: every load stays in bounds and no branch
  // splits the load pipeline.
  const int last_pos = first_pos + max(wave_hi - 1, 0);
  const int page_mask = a.page_size - 1;
  auto table_entry = [&](int tile) -> int32_t {
    const int pos = min(first_pos + tile + lane, last_pos);
    return tab[pos >> a.page_shift];
  };
  auto slot_from = [&](int32_t entry, int tile) -> uint32_t {
    const int pos = min(first_pos + tile + lane, last_pos);
    const uint32_t slot = ((uint32_t)entry << a.page_shift) + (uint32_t)(pos & page_mask);
    return slot < a.pool_rows ? slot : a.pool_rows - 1;
  };

  auto issue = [&](uint4 (&buf)[SB][KVS], uint32_t slots, int first_step) {
#pragma unroll
    for (int i = 0; i < SB; ++i) {
      const int step = first_step + i;
      uint32_t slot;
      if (TPW == 1) {
        slot = __builtin_amdgcn_readlane(slots, step);
      } else if (TPW == 2) {
        const uint32_t s0 = __builtin_amdgcn_readlane(slots, 2 * step);
        const uint32_t s1 = __builtin_amdgcn_readlane(slots, 2 * step + 1);
        slot = tok_sub ? s1 : s0;
      } else {
        const uint32_t s0 = __builtin_amdgcn_readlane(slots, 4 * step);
        const uint32_t s1 = __builtin_amdgcn_readlane(slots, 4 * step + 1);
        const uint32_t s2 = __builtin_amdgcn_readlane(slots, 4 * step + 2);
        const uint32_t s3 = __builtin_amdgcn_readlane(slots, 4 * step + 3);
        slot = tok_sub == 0 ? s0 : (tok_sub == 1 ? s1 : (tok_sub == 2 ? s2 : s3));
      }
      const char* row = (const char*)a.k_pool + (size_t)slot * (size_t)(HKV * kHeadDim * 2);
#pragma unroll
      for (int s = 0; s < KVS; ++s) {
        uint32_t off = kv_off[s];
        asm volatile("" : "+v"(off));  // keep the 32-bit lane offset next to its use
        buf[i][s] = *(const uint4*)(row + off);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  auto reduce = [&](const uint4 (&buf)[SB][KVS], float (&res)[KVS][G], int first_step) {
#pragma unroll
    for (int i = 0; i < SB; ++i) {
#pragma unroll
      for (int s = 0; s < KVS; ++s)
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const float p = row16_sum(dot8(buf[i][s], qreg[s][g]));
          res[s][g] = (l16 == first_step + i) ? p : res[s][g];
          // Pin the select here; otherwise the compiler sinks the whole chain
          // into the store block and keeps every partial sum alive until then.
          asm volatile("" : "+v"(res[s][g]));
        }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  uint32_t slots_cur = 0;
  if (wave_lo < wave_hi) {
    slots_cur = slot_from(table_entry(wave_lo), wave_lo);
    issue(buf0, slots_cur, 0);
  }

  for (int tile = wave_lo; tile < wave_hi; tile += TILE) {
    float res[KVS][G];
#pragma unroll
    for (int s = 0; s < KVS; ++s)
#pragma unroll
      for (int g = 0; g < G; ++g) res[s][g] = 0.f;

    const int32_t entry_next = table_entry(tile + TILE);
    uint32_t slots_next = 0;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int sb = 0; sb < NSB; sb += 2) {
      // buf0 holds sub-batch sb; fetch sb+1 into buf1, then sb+2 into buf0.
      issue(buf1, slots_cur, (sb + 1) * SB);
      reduce(buf0, res, sb * SB);
      if (sb + 2 < NSB) {
        issue(buf0, slots_cur, (sb + 2) * SB);
      } else {
        slots_next = slot_from(entry_next, tile + TILE);
        issue(buf0, slots_next, 0);
      }
      reduce(buf1, res, (sb + 1) * SB);
    }
    slots_cur = slots_next;

    // Lane l16 of each group now holds token tile + l16*TPW + tok_sub.
    const int mytok = tile + l16 * TPW + tok_sub;
    if (mytok < wave_hi) {
#pragma unroll
      for (int s = 0; s < KVS; ++s) {
        const int kvh = HKV >= 4 ? lg + 4 * s : lg % HKV;
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int h = head_of<HKV, G>(kvh, g, a.head_map);
          const float x = res[s][g];
          const size_t at = ((size_t)b * H + h) * (size_t)a.score_stride + (size_t)mytok;
          if (OUT_BF16)
            ((uint16_t*)a.scores)[at] = f32_to_bf16(x);
          else
            ((float*)a.scores)[at] = x;
          // Online (max, sum exp) with a single exponential per element.
          const float d = x - run_m[s][g];
          const float e = __expf(-fabsf(d));
          if (d > 0.f) {
            run_l[s][g] = run_l[s][g] * e + 1.f;
            run_m[s][g] = x;
          } else {
            run_l[s][g] += e;
          }
        }
      }
    }
  }

  if (a.partials == nullptr) return;

  __shared__ float sm_m[4][4][KVS][G];
  __shared__ float sm_l[4][4][KVS][G];
#pragma unroll
  for (int s = 0; s < KVS; ++s)
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float m = run_m[s][g], l = run_l[s][g];
      row16_softmax_merge(m, l);
      if (l16 == 0) {
        sm_m[wave][lg][s][g] = m;
        sm_l[wave][lg][s][g] = l;
      }
    }
  __syncthreads();
  if ((int)threadIdx.x < H) {
    const int h = threadIdx.x;
    float m = kNegBig, l = 0.f;
    for (int w = 0; w < 4; ++w)
      for (int gi = 0; gi < 4; ++gi)
        for (int s = 0; s < KVS; ++s) {
          const int kvh = HKV >= 4 ? gi + 4 * s : gi % HKV;
          for (int g = 0; g < G; ++g)
            if (head_of<HKV, G>(kvh, g, a.head_map) == h)
              softmax_merge(m, l, sm_m[w][gi][s][g], sm_l[w][gi][s][g]);
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
