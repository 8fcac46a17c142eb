// Criticality scoring: scores[h,t] = q[h,:] . K[slot(t), kv(h), :] streamed over the
// paged KV cache (the reference's paged_matmul_kernel, tr.py:166-231), plus the
// per-head softmax statistics the soft vote needs (tr.py:361).
//
// The pass is bound by HBM: every candidate row (Hkv*256 bytes) is read exactly
// once for all H query heads.  The dot products go through the matrix cores, not
// because the shape is a dense GEMM (it is 1 to 8 query rows per KV head) but
// because one v_mfma_f32_16x16x32_bf16 replaces some 64 dot / reduce / select
// vector instructions, which is what lets a wavefront keep 32 KB of loads in
// flight instead of computing.
//
// Operand layout (lane l: rg = l/16, t4 = (l%16)/4, p = l%4).  One load
// instruction covers four tokens of a tile and one KV head: lane l reads the 16
// bytes at offset 64*rg + 16*p of token 4m + t4, so each token's 256-byte head
// row is fetched as one contiguous piece and every 128-byte line is consumed by
// a single instruction.  Seen as the B operand (column l%16, k-group rg), column
// (t4, p) holds the dims {8(4rg + p) + e} of token t4: a quarter of the head
// dimension per column.  The A operand uses the same mapping with the query head
// in place of the token, so that D[(g, p'), (t4, p)] is the partial dot product
// of query g and token t4 over quarter p when p' == p.  Each lane keeps the
// diagonal element (register p of its 4 results) and the four quarters are added
// across the 4 lanes of a quad with two DPP quad_perm adds.  After the four
// instructions of a tile (m = 0..3) lane (rg, t4, p) keeps the result of m == p:
// the score of query rg for token 4p + t4, one token per lane, 16 tokens per
// 16-lane row, stored as one 64-byte segment per head.
//
// Products of bf16 pairs are exact in fp32 and the accumulation is fp32.
// Loads are double-buffered in half iterations (16 x 128-bit loads per lane
// each) and the table entries of the next iteration are fetched one iteration
// ahead.
#include <stdlib.h>

#include <atomic>

#include "ts_score.h"
#include "ts_topk.h"

namespace ts {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

template <int HKV, int G>
__device__ __forceinline__ int head_of(int kvh, int g, int head_map) {
  return head_map == TS_HEADMAP_MOD ? kvh + HKV * g : kvh * G + g;
}

// 128-bit load with the non-temporal hint: the keys are read once, and keeping
// them out of the caches' replacement order is worth about 10 % of streaming
// bandwidth on this part.
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
__device__ __forceinline__ uint4 load_streaming(const char* p) {
  const u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}

constexpr int kQuadSwap1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;  // quad_perm [2,3,0,1]

// One iteration of a wave covers TG tiles of 16 tokens and all HKV heads: always
// 8 (tile, KV head) units = 32 loads of 1 KB.  Units 0-3 and 4-7 alternate
// between two register buffers.
//
// Output forms:
//   kScoreDirect (paged_matmul): scores[h][t] row-major in the caller's dtype,
//     stored directly.
//   kScoreTiled (the selection path, separate kernels): fp32 scores leave the
//     kernel tile-major, scores[b][tile][head slot][16 tokens] with head slot =
//     kvh*G + g.  They are staged in LDS and written once per workgroup as one
//     contiguous burst: trickling 64-byte pieces into 32 separate head rows while
//     the keys stream in costs a quarter of the read bandwidth (DRAM read/write
//     turnarounds).
//   kScoreFused (score + vote in one launch whose workgroups are all resident at
//     once and meet twice): the scores never leave LDS.  Every workgroup publishes
//     its per-head (max, sum exp); after the first rendezvous the (request, head)
//     pairs are dealt out over the grid and merged; after the second every
//     workgroup turns its own scores into votes (tr.py:361) and into the first
//     histogram of the selection.
constexpr int kScoreDirect = 0, kScoreTiled = 1, kScoreFused = 2;
constexpr int kMaxHeads = 128;

// Data that workgroups of one launch hand to each other goes through
// device-coherent accesses (relaxed agent-scope atomics): the L2 of an XCD is not
// coherent with the other seven, and the fences that would make ordinary accesses
// visible write back and invalidate a whole L2 per workgroup, which costs several
// times the streaming pass itself.
__device__ __forceinline__ float2 load_coherent(const float2* p) {
  const uint64_t v =
      __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__uint_as_float((uint32_t)v), __uint_as_float((uint32_t)(v >> 32)));
}
__device__ __forceinline__ void store_coherent(float2* p, float m, float l) {
  const uint64_t v = (uint64_t)__float_as_uint(m) | ((uint64_t)__float_as_uint(l) << 32);
  __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Grid-wide rendezvous of a fully resident grid: every workgroup arrives once per
// round (1, 2, ...) and those that need the others' data wait for the round to
// complete.  Each thread first waits for its own coherent stores to be
// acknowledged; thread 0 then counts the workgroup in.  The workgroup that
// completes the count raises the round number in every replica slot, and the
// waiting ones poll the replica of their own index: hundreds of early workgroups
// polling one word would saturate the memory channel it lives in, which the
// workgroups still streaming need for 1/128 of their keys.  The wait is bounded:
// if the round does not complete within `ticks` of the 100 MHz clock the fault
// word is set and the workgroup carries on, so the kernel always drains.
__device__ __forceinline__ void grid_arrive(uint32_t* sync, bool wait, uint32_t round,
                                            uint64_t ticks) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t workgroups = gridDim.x * gridDim.y;
    const uint32_t index = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t before =
        __hip_atomic_fetch_add(&sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (before + 1 == round * workgroups) {
      for (int r = 0; r < kSyncSlots; ++r)
        __hip_atomic_store(&sync[(size_t)(r + 1) * kSyncSlotWords], round, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    } else if (wait) {
      const uint32_t* flag = &sync[(size_t)(index % kSyncSlots + 1) * kSyncSlotWords];
      const uint64_t t0 = wall_clock64();
      while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < round) {
        if (wall_clock64() - t0 > ticks) {
          __hip_atomic_store(&sync[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(16);
      }
    }
  }
  __syncthreads();
}

// Between the two rendezvous of the fused kernel: the (request, head) pairs are
// dealt out over all wavefronts of the grid; a wavefront merges the per-workgroup
// (max, sum exp) of its pair, a lane per chunk, in a fixed order.
__device__ __forceinline__ void merge_request_stats(const ScoreArgs& a, int lane, int wave) {
  const int H = a.num_heads;
  const int items = (int)gridDim.y * H;
  const int first = ((int)blockIdx.y * (int)gridDim.x + (int)blockIdx.x) * 4 + wave;
  const int step = (int)gridDim.x * (int)gridDim.y * 4;
  for (int item = first; item < items; item += step) {
    const int b = item / H, h = item % H;
    if (a.skip && a.skip[b]) continue;
    const ReqGeom geo =
        request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
    if (geo.n <= 0) continue;
    const int chunks = (geo.n + a.tokens_per_block - 1) / a.tokens_per_block;
    const float2* part = (const float2*)a.partials + ((size_t)b * H + h) * a.nchunks;
    float m = kNegBig, l = 0.f;
    for (int base = 0; base < chunks; base += 8 * 64) {  // 8 loads in flight per lane
      float2 v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int c = base + 64 * i + lane;
        v[i] = c < chunks ? load_coherent(part + c) : make_float2(kNegBig, 0.f);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) softmax_merge(m, l, v[i].x, v[i].y);
    }
    row16_softmax_merge(m, l);
    softmax_merge(m, l, __shfl_xor(m, 16), __shfl_xor(l, 16));
    softmax_merge(m, l, __shfl_xor(m, 32), __shfl_xor(l, 32));
    if (lane == 0) store_coherent((float2*)a.stats + (size_t)b * H + h, m, l);
  }
}

template <int HKV, int G, bool OUT_BF16, int MODE>
__global__ __launch_bounds__(256, (G > 4 ? 1 : 2)) void score_kernel(ScoreArgs a) {
  extern __shared__ float stage[];  // tiled / fused: [tiles of the workgroup][tile_stride]
  constexpr bool TILED = MODE != kScoreDirect;
  constexpr int TG = 8 / HKV;
  constexpr int UNITS = 8;
  constexpr int HALF = UNITS / 2;
  constexpr int NA = (G + 3) / 4;  // A operands (4 query heads each) per KV head
  constexpr int ITER = 16 * TG;    // tokens per iteration
  constexpr uint32_t ROW_BYTES = HKV * kHeadDim * 2;

  const int b = blockIdx.y;
  int n, first_pos;
  if (a.direct_n >= 0) {
    n = (int)a.direct_n;
    first_pos = 0;
  } else {
    ReqGeom geo = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k,
                                   a.max_seq_len);
    n = (a.skip && a.skip[b]) ? 0 : geo.n;
    first_pos = a.n_init;
  }
  const int block_lo = blockIdx.x * a.tokens_per_block;
  if (block_lo >= n) {
    if constexpr (MODE == kScoreFused) {  // no tokens here: only help with the statistics
      grid_arrive(a.sync, true, 1, a.spin_ticks);
      merge_request_stats(a, threadIdx.x & 63, threadIdx.x >> 6);
      grid_arrive(a.sync, false, 2, a.spin_ticks);
    }
    return;
  }

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rg = lane >> 4;        // k-group of the operands, row group of the result
  const int t4 = (lane & 15) >> 2;  // token of a 4-token group / query of a 4-query group
  const int p = lane & 3;           // quarter of the head dimension
  const uint32_t lane_off = (uint32_t)(rg * 64 + p * 16);
  const int H = a.num_heads;
  // Fused: one spare row per tile keeps the four tiles a wavefront reads in the
  // vote phase on different LDS banks.
  const int tile_stride = MODE == kScoreFused ? 16 * H + 16 : 16 * H;
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;

  // A operands: query 4*na + t4 of each KV head, same byte offsets as the keys.
  bf16x8_t qa[HKV][NA];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      const int g = 4 * na + t4;
      const int h = head_of<HKV, G>(kvh, g < G ? g : 0, a.head_map);
      uint4 v = *(const uint4*)((const char*)(a.qf + ((size_t)b * H + h) * kHeadDim) + lane_off);
      if (g >= G) v = make_uint4(0u, 0u, 0u, 0u);
      qa[kvh][na] = __builtin_bit_cast(bf16x8_t, v);
    }

  float run_m[HKV][NA], run_l[HKV][NA];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      run_m[kvh][na] = kNegBig;
      run_l[kvh][na] = 0.f;
    }

  const int per_wave = a.tokens_per_block >> 2;
  const int wave_lo = block_lo + wave * per_wave;
  const int wave_hi = min(wave_lo + per_wave, n);

  // Lane (rg, t4, p) addresses tokens tile + 4m + t4, m = 0..3, of every tile.
  // The table loads and the slot arithmetic are split so that the entries of the
  // next iteration are requested a whole iteration before they are needed.
  // Positions past the wave's range are clamped to its last token: every load
  // stays in bounds and no branch splits the load pipeline.
  const int last_pos = first_pos + max(wave_hi - 1, 0);
  const int page_mask = a.page_size - 1;
  auto table_entry = [&](int tok) -> int32_t {
    const int pos = min(first_pos + tok, last_pos);
    return tab[pos >> a.page_shift];
  };
  // Byte offset of this lane's 16 bytes inside the pool.  Offsets, not pointers,
  // are carried across iterations: a pointer rebuilt from the kernel argument at
  // the load is known to be global memory, whereas a loop-carried pointer decays
  // to a flat access, whose completion the wave must wait for in full.
  auto row_off = [&](int32_t entry, int tok) -> size_t {
    const int pos = min(first_pos + tok, last_pos);
    uint32_t slot = ((uint32_t)entry << a.page_shift) + (uint32_t)(pos & page_mask);
    slot = slot < a.pool_rows ? slot : a.pool_rows - 1;
    return (size_t)slot * ROW_BYTES + lane_off;
  };
  const char* const pool = (const char*)a.k_pool;

  // Lane-constant bit masks: all ones where p == i.  Selecting with and/or keeps
  // the loop free of branches (a ternary chain on p is lowered to a switch).
  uint32_t pmask[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    pmask[i] = p == i ? 0xffffffffu : 0u;
    asm volatile("" : "+v"(pmask[i]));
  }

  uint4 buf0[HALF][4], buf1[HALF][4];
  auto issue = [&](uint4 (&buf)[HALF][4], auto& rows, int first_unit) {
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
      const int u = first_unit + i;
#pragma unroll
      for (int m = 0; m < 4; ++m)
        buf[i][m] = load_streaming(pool + rows[u / HKV][m] + (u % HKV) * (kHeadDim * 2));
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // res[u][na]: score of query 4*na + rg (of the unit's KV head) for token
  // tile + 4p + t4.
  auto multiply = [&](const uint4 (&buf)[HALF][4], float (&res)[UNITS][NA], int first_unit) {
#pragma unroll
    for (int i = 0; i < HALF; ++i) {
      const int u = first_unit + i;
#pragma unroll
      for (int na = 0; na < NA; ++na) {
        uint32_t keep = 0u;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
          const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
          const f32x4_t d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              qa[u % HKV][na], __builtin_bit_cast(bf16x8_t, buf[i][m]), zero, 0, 0, 0);
          float v = __uint_as_float((__float_as_uint(d[0]) & pmask[0]) | (__float_as_uint(d[1]) & pmask[1]) |
                                    (__float_as_uint(d[2]) & pmask[2]) | (__float_as_uint(d[3]) & pmask[3]));
          v += dpp_move<kQuadSwap1>(v);
          v += dpp_move<kQuadSwap2>(v);
          keep |= __float_as_uint(v) & pmask[m];
        }
        res[u][na] = __uint_as_float(keep);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  size_t rows_cur[TG][4];
  size_t rows_next[TG][4];
  if (wave_lo < wave_hi) {
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const int tok = wave_lo + 16 * t + 4 * m + t4;
        rows_cur[t][m] = row_off(table_entry(tok), tok);
      }
    issue(buf0, rows_cur, 0);
  }

  for (int base = wave_lo; base < wave_hi; base += ITER) {
    int32_t entry_next[TG][4];
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
      for (int m = 0; m < 4; ++m) entry_next[t][m] = table_entry(base + ITER + 16 * t + 4 * m + t4);
    __builtin_amdgcn_sched_barrier(0);

    float res[UNITS][NA];
    issue(buf1, rows_cur, HALF);
    multiply(buf0, res, 0);
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
      for (int m = 0; m < 4; ++m)
        rows_next[t][m] = row_off(entry_next[t][m], base + ITER + 16 * t + 4 * m + t4);
    issue(buf0, rows_next, 0);
    multiply(buf1, res, HALF);
#pragma unroll
    for (int t = 0; t < TG; ++t)
#pragma unroll
      for (int m = 0; m < 4; ++m) rows_cur[t][m] = rows_next[t][m];

#pragma unroll
    for (int u = 0; u < UNITS; ++u) {
      const int t = u / HKV, kvh = u % HKV;
      const int tok = base + 16 * t + 4 * p + t4;
#pragma unroll
      for (int na = 0; na < NA; ++na) {
        const int g = 4 * na + rg;
        if (g < G && tok < wave_hi) {
          const int h = head_of<HKV, G>(kvh, g, a.head_map);
          const float x = res[u][na];
          if (TILED) {
            stage[((tok - block_lo) >> 4) * tile_stride + (kvh * G + g) * 16 + (tok & 15)] = x;
          } else {
            const size_t at = ((size_t)b * H + h) * (size_t)a.score_stride + (size_t)tok;
            if (OUT_BF16)
              ((uint16_t*)a.scores)[at] = f32_to_bf16(x);
            else
              ((float*)a.scores)[at] = x;
          }
          // Online (max, sum exp) with a single exponential per element.
          const float d = x - run_m[kvh][na];
          const float e = __expf(-fabsf(d));
          if (d > 0.f) {
            run_l[kvh][na] = run_l[kvh][na] * e + 1.f;
            run_m[kvh][na] = x;
          } else {
            run_l[kvh][na] += e;
          }
        }
      }
    }
  }

  if (MODE == kScoreTiled) {  // one contiguous burst per workgroup
    __syncthreads();
    const int tiles = (min(a.tokens_per_block, n - block_lo) + 15) >> 4;
    float4* dst = (float4*)((float*)a.scores + ((size_t)b * a.score_stride + block_lo) * H);
    const float4* src = (const float4*)stage;
    for (int i = threadIdx.x; i < tiles * H * 4; i += 256) dst[i] = src[i];
  }
  if (a.partials == nullptr) return;

  // Per-workgroup (max, sum exp) of every head: 16 lanes of a row, then 4 waves.
  __shared__ float sm_m[4][4][HKV][NA];
  __shared__ float sm_l[4][4][HKV][NA];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      float m = run_m[kvh][na], l = run_l[kvh][na];
      row16_softmax_merge(m, l);
      if ((lane & 15) == 0) {
        sm_m[wave][rg][kvh][na] = m;
        sm_l[wave][rg][kvh][na] = l;
      }
    }
  __syncthreads();
  if ((int)threadIdx.x < 4 * HKV * NA) {
    const int na = threadIdx.x % NA;
    const int kvh = (threadIdx.x / NA) % HKV;
    const int g4 = threadIdx.x / (NA * HKV);
    const int g = 4 * na + g4;
    if (g < G) {
      float m = sm_m[0][g4][kvh][na], l = sm_l[0][g4][kvh][na];
#pragma unroll
      for (int w = 1; w < 4; ++w) softmax_merge(m, l, sm_m[w][g4][kvh][na], sm_l[w][g4][kvh][na]);
      const int h = head_of<HKV, G>(kvh, g, a.head_map);
      float2* out = (float2*)a.partials + ((size_t)b * H + h) * a.nchunks + blockIdx.x;
      if (MODE == kScoreFused)
        store_coherent(out, m, l);
      else
        *out = make_float2(m, l);
    }
  }

  if constexpr (MODE == kScoreFused) {
    __shared__ float s_max[kMaxHeads];
    __shared__ float s_rz[kMaxHeads];
    __shared__ uint32_t lh[kTopkBins];
    for (int i = threadIdx.x; i < kTopkBins; i += 256) lh[i] = 0u;
    grid_arrive(a.sync, true, 1, a.spin_ticks);
    merge_request_stats(a, lane, wave);
    grid_arrive(a.sync, true, 2, a.spin_ticks);
    for (int slot = threadIdx.x; slot < H; slot += 256) {
      const int h = head_of<HKV, G>(slot / G, slot % G, a.head_map);
      const float2 st = load_coherent((const float2*)a.stats + (size_t)b * H + h);
      s_max[slot] = st.x;
      s_rz[slot] = 1.0f / st.y;
    }
    __syncthreads();

    // Votes of this workgroup's tokens: fp32 sum over the head slots in slot order.
    const int count = min(a.tokens_per_block, n - block_lo);
    for (int i = threadIdx.x; i < count; i += 256) {
      const float* sc = stage + (i >> 4) * tile_stride + (i & 15);
      float c = 0.f;
      for (int slot = 0; slot < H; ++slot) c += __expf(sc[slot * 16] - s_max[slot]) * s_rz[slot];
      a.votes[(size_t)b * a.vote_stride + block_lo + i] = c;
      atomicAdd(&lh[key_bin0(vote_key(c))], 1u);
    }
    __syncthreads();
    uint32_t* hist0 = hist0_copy(topk_ws(a.topk_ws, a.topk_ws_stride, b), blockIdx.x);
    for (int i = threadIdx.x; i < kTopkBins; i += 256)
      if (lh[i]) atomicAdd(&hist0[i], lh[i]);
  }
}

template <bool OUT_BF16, int MODE>
static int launch_score(int hkv, int group, const ScoreArgs& a, dim3 grid, hipStream_t stream) {
  const size_t lds =
      MODE == kScoreTiled ? (size_t)a.tokens_per_block * a.num_heads * sizeof(float) : 0;
#define TS_SCORE_CASE(HKV_, G_)                                                                  \
  if (hkv == HKV_ && group == G_) {                                                              \
    hipLaunchKernelGGL((score_kernel<HKV_, G_, OUT_BF16, MODE>), grid, dim3(256), lds, stream, a); \
    return check_launch("score_kernel");                                                         \
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

// The fused kernel of a head shape, or NULL.
static const void* fused_kernel_of(int hkv, int group) {
#define TS_SCORE_CASE(HKV_, G_) \
  if (hkv == HKV_ && group == G_) return (const void*)&score_kernel<HKV_, G_, false, kScoreFused>;
#define TS_SCORE_ROW(HKV_) \
  TS_SCORE_CASE(HKV_, 1) TS_SCORE_CASE(HKV_, 2) TS_SCORE_CASE(HKV_, 4) TS_SCORE_CASE(HKV_, 7) TS_SCORE_CASE(HKV_, 8)
  TS_SCORE_ROW(1)
  TS_SCORE_ROW(2)
  TS_SCORE_ROW(4)
  TS_SCORE_ROW(8)
#undef TS_SCORE_ROW
#undef TS_SCORE_CASE
  return nullptr;
}

static size_t fused_lds_bytes(int tokens_per_block, int num_heads) {
  return (size_t)(tokens_per_block / 16) * (16 * num_heads + 16) * sizeof(float);
}

// Dynamic LDS the fused form may use: with the 10 KB of static arrays, two
// workgroups fit the 160 KB of a CU.
constexpr size_t kFusedStageBytes = 68 * 1024;

static std::atomic<int> g_fused_vote{[] {
  const char* e = getenv("TS_FUSED_VOTE");  // "0" starts with the separate kernels
  return (e && e[0] == '0') ? 0 : 1;
}()};

int set_fused_vote(int enable) { return g_fused_vote.exchange(enable ? 1 : 0); }

int fused_tokens_per_block(const ts_config* cfg, int batch, int max_seq_len) {
  if (!g_fused_vote.load() || cfg->pool_kernel > 0 || cfg->num_heads > kMaxHeads) return 0;
  const int max_n = max_seq_len - cfg->n_init - cfg->n_local;
  if (max_n <= 0) return 0;
  const int group = cfg->num_heads / cfg->num_kv_heads;
  const void* fn = fused_kernel_of(cfg->num_kv_heads, group);
  if (!fn) return 0;

  // Workgroups the device keeps resident at once; depends on the kernel only.
  struct Entry { const void* fn; int device; int capacity; };
  static thread_local Entry memo[4] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  int capacity = 0;
  for (const Entry& e : memo)
    if (e.fn == fn && e.device == device) capacity = e.capacity;
  if (capacity == 0) {
    int per_cu = 0, cus = 0;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFusedStageBytes) !=
        hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 256, kFusedStageBytes) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    capacity = per_cu * cus;
    if (capacity <= 0) return 0;
    static thread_local int next = 0;
    memo[next++ % 4] = Entry{fn, device, capacity};
  }

  int tpb = score_tokens_per_block((int64_t)batch * max_seq_len, cfg->num_heads);
  while ((int64_t)ceil_div(max_n, tpb) * batch > capacity) tpb += 64;
  if (fused_lds_bytes(tpb, cfg->num_heads) > kFusedStageBytes) return 0;
  return tpb;
}

// Bytes of the per-workgroup partials proper; the merged statistics of the fused
// kernel follow them.
static size_t partials_region_bytes(const ts_config* cfg, int batch, size_t nchunks) {
  return align_up((size_t)batch * cfg->num_heads * nchunks * 2 * sizeof(float), 256);
}

static ScoreArgs selection_args(const ts_config* cfg, const ts_batch* bt, const void* qf,
                                const void* k_pool, int64_t pool_rows, const int32_t* skip,
                                float* partials, int tokens_per_block) {
  ScoreArgs a{};
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
  a.partials = partials;
  a.tokens_per_block = tokens_per_block;
  a.nchunks = (int)ceil_div(bt->max_seq_len, tokens_per_block);
  a.num_heads = cfg->num_heads;
  a.head_map = cfg->head_map;
  return a;
}

}  // namespace ts

using namespace ts;

extern "C" {

int ts_set_fused_vote(int enable) { return set_fused_vote(enable); }

size_t ts_score_partials_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  const int tpb = score_tokens_per_block((int64_t)batch * max_seq_len, cfg->num_heads);
  const size_t nchunks = (size_t)ceil_div(max_seq_len, tpb);
  return partials_region_bytes(cfg, batch, nchunks) +
         align_up((size_t)batch * cfg->num_heads * 2 * sizeof(float), 256);  // + merged statistics
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
  TS_REQUIRE(score_stride >= max_n && score_stride >= 16 && score_stride % 16 == 0, TS_EWORKSPACE,
             "score_stride %lld must be a multiple of 16 and >= max candidates %d",
             (long long)score_stride, max_n);
  const size_t need = ts_score_partials_bytes(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(partials_bytes >= need, TS_EWORKSPACE, "ts_score: partials %zu bytes < required %zu",
             partials_bytes, need);
  if (max_n <= 0) return TS_OK;  // every request is dense

  ScoreArgs a = selection_args(
      cfg, bt, qf, k_pool, pool_rows, skip, partials,
      score_tokens_per_block((int64_t)bt->batch * bt->max_seq_len, cfg->num_heads));
  a.scores = scores;
  a.score_stride = score_stride;
  const dim3 grid((unsigned)ceil_div(max_n, a.tokens_per_block), (unsigned)bt->batch);
  return launch_score<false, kScoreTiled>(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads, a, grid,
                                   (hipStream_t)stream);
}

int ts_score_vote_supported(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  return fused_tokens_per_block(cfg, batch, max_seq_len) > 0 ? 1 : 0;
}

int ts_score_vote(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                  int64_t pool_rows, const int32_t* skip, float* votes, int64_t vote_stride,
                  float* partials, size_t partials_bytes, void* topk_workspace,
                  size_t topk_workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(qf && k_pool && votes && partials && topk_workspace, TS_EINVAL,
             "ts_score_vote: NULL tensor argument");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  TS_REQUIRE(partials_bytes >= ts_score_partials_bytes(cfg, bt->batch, bt->max_seq_len),
             TS_EWORKSPACE, "ts_score_vote: partials %zu bytes too small", partials_bytes);
  TS_REQUIRE(topk_workspace_bytes >= ts_topk_workspace_bytes(cfg, bt->batch, bt->max_seq_len),
             TS_EWORKSPACE, "ts_score_vote: top-k workspace %zu bytes too small",
             topk_workspace_bytes);
  const int tpb = fused_tokens_per_block(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(tpb > 0, TS_ESHAPE,
             "ts_score_vote: batch %d x %d tokens does not fit one co-resident grid (or pool_kernel "
             "is on); use ts_score + ts_vote",
             bt->batch, bt->max_seq_len);

  ScoreArgs a = selection_args(cfg, bt, qf, k_pool, pool_rows, skip, partials, tpb);
  const int unfused_tpb =
      score_tokens_per_block((int64_t)bt->batch * bt->max_seq_len, cfg->num_heads);
  a.stats = (float*)((char*)partials +
                     partials_region_bytes(cfg, bt->batch, ceil_div(bt->max_seq_len, unfused_tpb)));
  a.votes = votes;
  a.vote_stride = vote_stride;
  a.topk_ws = (uint32_t*)topk_workspace;
  a.topk_ws_stride = topk_ws_stride_words(max_n);
  a.sync = topk_sync_area(topk_workspace, bt->batch, max_n);
  a.spin_ticks = 200000000ull;  // 2 s of the 100 MHz clock
  const void* fn = fused_kernel_of(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads);
  const dim3 grid((unsigned)ceil_div(max_n, tpb), (unsigned)bt->batch);
  void* params[] = {(void*)&a};
  // An ordinary launch: the grid was sized to be resident all at once, which holds
  // as long as the device runs nothing else beside this stream.  (The cooperative
  // launch API would guarantee it, at some 25 us of extra launch latency.)
  const hipError_t e = hipLaunchKernel(fn, grid, dim3(256), params,
                                       fused_lds_bytes(tpb, cfg->num_heads), (hipStream_t)stream);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(TS_EHIP, "ts_score_vote launch: %s", hipGetErrorString(e));
  }
  return TS_OK;
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

  ScoreArgs a{};
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
  a.tokens_per_block = score_tokens_per_block(n, num_heads);
  a.nchunks = (int)ceil_div(n, a.tokens_per_block);
  a.num_heads = num_heads;
  a.head_map = TS_HEADMAP_MOD;
  const dim3 grid((unsigned)a.nchunks, 1);
  if (scores_dtype == TS_DTYPE_BF16)
    return launch_score<true, kScoreDirect>(num_kv_heads, num_heads / num_kv_heads, a, grid,
                                     (hipStream_t)stream);
  return launch_score<false, kScoreDirect>(num_kv_heads, num_heads / num_kv_heads, a, grid,
                                    (hipStream_t)stream);
}

}  // extern "C"
