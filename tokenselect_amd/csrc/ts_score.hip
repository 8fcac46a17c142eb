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

#include <algorithm>
#include <atomic>
#include <vector>

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
//   kScoreFused (the whole selection in one launch whose workgroups are all
//     resident at once and meet two to four times): the scores never leave LDS.
//     Every workgroup publishes its per-head (max, sum exp); the (request, head)
//     pairs are dealt out over the grid, merged and written to replicas that the
//     workgroups poll; every workgroup turns its own
//     scores into votes (tr.py:361); histogram rounds (11 + 11 + 10 key bits) narrow
//     the k-th largest vote down until at most 256 candidates are left, which are
//     listed and ranked by every workgroup together with the counts that tell it
//     where its selected positions, in ascending order, belong (tr.py:371-373,
//     433-449); masses of exact ties go through all three levels and a count round.
constexpr int kScoreDirect = 0, kScoreTiled = 1, kScoreFused = 2;
// The fused kernel's votes-only form (phases of requests in one launch): a kernel of its
// own, so that the single-launch selection does not carry the bookkeeping.
constexpr int kScorePacked = 3;
constexpr int kMaxHeads = 128;

// What a workgroup of the fused kernel serves: the whole launch, or one phase of a
// launch of the votes-only form.
struct LaunchPart {
  int tokens_per_block;
  int batch_offset;       // first request
  int packed;             // requests of the phase (0: the grid is [chunks, requests])
  const int* pack_first;  // first workgroup of each of them
  int x;                  // this workgroup along x
  uint32_t* sync;         // rendezvous area
};

// Chunks of request r of a phase that hold candidates: those of its n candidates, but no
// more than the phase has workgroups for it (a length above the bound the phase was sized
// by is the caller's error: the tokens beyond are not scored, and the launch reports it).
__device__ __forceinline__ int packed_chunks(const LaunchPart& lp, int r, int n) {
  const int chunks = (n + lp.tokens_per_block - 1) / lp.tokens_per_block;
  return min(chunks, lp.pack_first[r + 1] - lp.pack_first[r]);
}

// The softmax statistics of the fused kernel, without a rendezvous: every workgroup
// publishes its per-head (max, sum exp) into a table that was zero at launch; the
// (request, head) pairs are dealt out over all wavefronts of the team; a wavefront polls
// the entries of its pair, a lane per chunk, until none is zero any more (a sum of
// exponentials never is: the data is its own flag), merges them in a fixed order and
// writes the result into 64 replicas, lane r into replica r.  The workgroups poll the
// words of the replica of their index in the same way.  The wait is bounded like those
// of the rendezvous: on giving up it sets the fault word and merges what is there.
template <bool PACKED>
__device__ __forceinline__ void merge_request_stats(const ScoreArgs& a, const LaunchPart& lp,
                                                    const GridTeam& team, int lane, int wave) {
  const int H = a.num_heads;
  const int items = (PACKED ? lp.packed : a.batch) * H;
  const int first = (int)team.index * 4 + wave;
  const int step = (int)team.size * 4;
  for (int item = first; item < items; item += step) {
    const int b = lp.batch_offset + item / H, h = item % H;
    if (a.skip && a.skip[b]) continue;
    const ReqGeom geo =
        request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
    if (geo.n <= 0) continue;
    const int chunks = PACKED ? packed_chunks(lp, item / H, geo.n)
                              : (geo.n + lp.tokens_per_block - 1) / lp.tokens_per_block;
    const float2* part = (const float2*)a.partials + ((size_t)b * H + h) * a.nchunks;
    float m = kNegBig, l = 0.f;
    const uint64_t t0 = wall_clock64();
    bool lost = false;
    for (int base = 0; base < chunks; base += 8 * 64) {  // 8 loads in flight per lane
      float2 v[8];
      for (uint32_t polls = 1;; ++polls) {
        bool there = true;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int c = base + 64 * i + lane;
          v[i] = c < chunks ? load_coherent(part + c) : make_float2(kNegBig, 1.f);
          there = there && __float_as_uint(v[i].y) != 0u;
        }
        if (__all(there) || lost) break;
        if ((polls & 7u) == 0) {
          if (load_coherent(&lp.sync[0]) != 0u) {
            lost = true;
          } else if (wall_clock64() - t0 > a.spin_ticks) {
            __hip_atomic_store(&lp.sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            lost = true;
          }
        }
        __builtin_amdgcn_s_sleep(8);  // some 0.2 us between the polls of a few dozen wavefronts
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int c = base + 64 * i + lane;
        if (c < chunks) softmax_merge(m, l, v[i].x, v[i].y);
      }
    }
    row16_softmax_merge(m, l);
    softmax_merge(m, l, __shfl_xor(m, 16), __shfl_xor(l, 16));
    softmax_merge(m, l, __shfl_xor(m, 32), __shfl_xor(l, 32));
    store_coherent((float2*)(a.stats + (size_t)lane * a.stats_stride) + (size_t)b * H + h, m, l);
  }
}

constexpr int kStatsPollSleep = 12;     // x 64 clocks between a workgroup's polls for the merged statistics
constexpr uint32_t kSelectRounds = 4;  // rendezvous of the fused kernel at most (without the max-pool's)

#ifdef TS_TRACE  // development builds only: per-workgroup phase timestamps of the fused kernel
#include "ts_trace.h"
#else
#define TS_MARK(i) \
  do {             \
  } while (0)
#endif

// The workgroups that take part in the rendezvous of the fused kernel: all those of
// the requests that select (neither dense nor served by the selection cache).  The
// others write their fixed output and leave, so that a step in which every request
// hits the cache costs a few microseconds instead of empty rounds.
// (req, chunk: this workgroup's request within the launch and its chunk of that request.)
template <bool PACKED>
__device__ __forceinline__ GridTeam selecting_team(const ScoreArgs& a, const LaunchPart& lp,
                                                   uint32_t* lds, int req, int chunk) {
  GridTeam team{0u, 0u};
  if (PACKED) {
    // A phase holds a handful of requests and its members are the workgroups
    // that hold candidates: every thread adds them up for itself.
    uint32_t before = 0, total = 0;
    for (int r = 0; r < lp.packed; ++r) {
      const int b = lp.batch_offset + r;
      if (a.skip && a.skip[b]) continue;
      const int n = request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k,
                                     a.max_seq_len).n;
      const uint32_t members = n > 0 ? (uint32_t)packed_chunks(lp, r, n) : 0u;
      total += members;
      if (r < req) before += members;
    }
    team.size = total + a.absent;
    team.index = before + (uint32_t)chunk;
    return team;
  }
  (void)lds;
  return team;  // (the single launch deals its workgroups itself: deal_workgroups)
}

// The single-launch selection deals its workgroups on the device, from the lengths and the
// hit flags as they are at launch: only the requests that select (neither dense nor served
// by the selection cache) get workgroups, all of them the same number of tokens, the
// smallest multiple of 64 with which the requests' chunks fit the grid; consecutive
// workgroups serve consecutive chunks, request after request.  A step in which one request
// of four misses the cache thus streams that request's keys through the whole device
// instead of through the quarter a fixed [chunks, requests] grid would give it, and a
// ragged batch is spread by what the requests hold, not by the longest.  Workgroups past
// the last chunk have nothing to do.  The workgroups with tokens are the team of the
// rendezvous, in grid order.
struct Deal {
  int tokens_per_block;  // of every selecting request of this launch
  int req;               // this workgroup's request (within the launch), -1: none
  int chunk, chunks;     // its chunk of that request, and the request's chunks
  uint32_t team_size, team_index;
};
constexpr int kDealPerLane = 8;  // requests per lane of the dealing wavefront: batches of up to 512

__device__ __forceinline__ int wave_sum(int x) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off);
  return x;
}

__device__ __forceinline__ Deal deal_workgroups(const ScoreArgs& a, int* lds) {
  const int tid = threadIdx.x, lane = tid & 63;
  const int B = a.batch, T = (int)gridDim.x, w = (int)blockIdx.x;
  if (B == 1) {  // one request: every thread works it out for itself, no exchange
    Deal d{a.tokens_per_block, -1, 0, 0, a.absent, (uint32_t)w};
    int n = 0;
    if (!(a.skip && a.skip[a.batch_offset]))
      n = request_geometry(a.seq_lens, a.k_per_req, a.batch_offset, a.n_init, a.n_local, a.top_k,
                           a.max_seq_len).n;
    if (n <= 0) return d;
    int tpb = max((n + T * 64 - 1) / (T * 64) * 64, 64);
    while ((n + tpb - 1) / tpb > T && tpb < a.tokens_per_block) tpb += 64;
    d.tokens_per_block = tpb;
    d.chunks = (n + tpb - 1) / tpb;
    d.team_size = (uint32_t)d.chunks + a.absent;
    if (w < d.chunks) {
      d.req = 0;
      d.chunk = w;
    }
    return d;
  }
  if (tid < 64) {
    // Request lane + 64 j: its candidates if it selects, else 0.
    int n[kDealPerLane];
    int all = 0;  // (what one launch holds fits the LDS of the device: far below 2^31)
#pragma unroll
    for (int j = 0; j < kDealPerLane; ++j) {
      const int b = lane + 64 * j;
      n[j] = 0;
      if (64 * j < B && b < B && !(a.skip && a.skip[a.batch_offset + b]))
        n[j] = request_geometry(a.seq_lens, a.k_per_req, a.batch_offset + b, a.n_init, a.n_local, a.top_k,
                                a.max_seq_len).n;
      all += n[j];
    }
    const long long total_n = wave_sum(all);
    // Fewest tokens per workgroup that could do, then upwards until the chunks fit (a step
    // or two: the rounding of every request's last chunk).  The launch's own figure always
    // fits: the host sized the grid for every request at the longest length.
    int tpb = (int)((total_n + (long long)T * 64 - 1) / ((long long)T * 64)) * 64;
    tpb = max(tpb, 64);
    int chunks[kDealPerLane];
    for (;; tpb += 64) {
      int mine = 0;
#pragma unroll
      for (int j = 0; j < kDealPerLane; ++j) {
        chunks[j] = 64 * j < B ? (n[j] + tpb - 1) / tpb : 0;
        mine += chunks[j];
      }
      if (wave_sum(mine) <= T || tpb >= a.tokens_per_block) break;
    }
    // First workgroup of every request, in request order (lane + 64 j: j by j).
    int base = 0, req = -1, chunk = 0, req_chunks = 0;
#pragma unroll
    for (int j = 0; j < kDealPerLane; ++j) {
      if (64 * j >= B) break;
      int incl = chunks[j];
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(incl, off);
        if (lane >= off) incl += up;
      }
      const int first = base + incl - chunks[j];
      const bool here = w >= first && w < first + chunks[j];
      const uint64_t who = __ballot(here);
      if (who) {
        const int src = __ffsll((unsigned long long)who) - 1;
        req = 64 * j + src;
        chunk = w - __shfl(first, src);
        req_chunks = __shfl(chunks[j], src);
      }
      base += __shfl(incl, 63);
    }
    if (lane == 0) {
      lds[0] = tpb;
      lds[1] = req;
      lds[2] = chunk;
      lds[3] = req_chunks;
      lds[4] = base;  // workgroups with tokens: the team
    }
  }
  __syncthreads();
  Deal d;
  d.tokens_per_block = lds[0];
  d.req = lds[1];
  d.chunk = lds[2];
  d.chunks = lds[3];
  d.team_size = (uint32_t)lds[4] + a.absent;
  d.team_index = (uint32_t)w;
  __syncthreads();
  return d;
}

// The parts of the output that need no votes, written while the keys stream: a
// dense request gets all its positions and a selection-cache hit its cached ones
// (both spread over the request's workgroups); workgroup 0 of a request writes the
// length, the sink and the local window, and clears the words the next kernel of
// the stream wants cleared.
// (x of nx: this workgroup among those that write the request's fixed parts.)
__device__ __forceinline__ void fixed_segments(const ScoreArgs& a, int b, int x, int nx) {
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;
  int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
  int32_t* sel_pos = a.sel_pos + (int64_t)b * a.sel_stride;
  const int L = geo.seq_len;
  const int first = x * 256 + threadIdx.x, step = nx * 256;
  auto emit = [&](int out_idx, int pos) {
    sel_pos[out_idx] = pos;
    sel[out_idx] = (int32_t)lookup_slot(tab, pos, a.page_size, a.page_shift, a.pool_rows);
  };
  if (x == 0 && a.clear)
    for (int i = threadIdx.x; i < a.clear_per_req; i += 256)
      a.clear[(size_t)b * a.clear_per_req + i] = 0u;
  if (geo.dense) {  // tr.py:377-378, 741-744: attend over every token
    for (int i = first; i < L; i += step) emit(i, i);
    if (first == 0) a.sel_len[b] = L;
    return;
  }
  const bool is_hit = a.skip && a.skip[b];
  const int k = is_hit ? min(a.cache_len[b], a.top_k) : geo.k;
  if (is_hit) {  // tr.py:419: reuse the cached positions
    const int32_t* cached = a.topk_cache + (int64_t)b * a.top_k;
    for (int i = first; i < k; i += step) emit(a.n_init + i, cached[i]);
  }
  if (x != 0) return;
  if (threadIdx.x == 0) {
    // (The length of a request that selects is written when its selection is through, by
    // the workgroup that also reports a wait that gave up: one writer, one order.)
    if (is_hit) a.sel_len[b] = a.n_init + k + a.n_local;
    if (!is_hit && a.cache_len) a.cache_len[b] = k;
  }
  for (int i = threadIdx.x; i < a.n_init; i += 256) emit(i, i);
  for (int i = threadIdx.x; i < a.n_local; i += 256) emit(a.n_init + k + i, L - a.n_local + i);
}

// Adds the wavefront's candidates to a histogram in memory with one fetch-add per
// distinct bin: normally a wavefront has a few candidates in different bins, but
// nearly uniform votes (a query of small norm) put all 64 lanes, of every wavefront,
// into the same bin, and that many single increments of one address take
// milliseconds.  Returns the old values (to be awaited).  Every lane of the wavefront
// must call it.
__device__ __forceinline__ uint32_t wave_histogram_add(uint32_t* hist, bool have, uint32_t bin,
                                                      int lane) {
  uint32_t done = 0;
  uint64_t todo = __ballot(have);
  while (todo) {
    const int leader = __ffsll((unsigned long long)todo) - 1;
    const uint32_t leader_bin = (uint32_t)__shfl((int)bin, leader);
    const uint64_t same = __ballot(have && bin == leader_bin) & todo;
    // Little sharing: the remaining lanes add on their own, in one instruction (a
    // wavefront whose 64 candidates sit in 64 bins must not issue 64 of them).
    if (__popcll(same) < 4) break;
    if (lane == leader) done += fetch_add_coherent(&hist[leader_bin], (uint32_t)__popcll(same));
    todo &= ~same;
  }
  if ((todo >> lane) & 1ull) done += fetch_add_coherent(&hist[bin], 1u);
  return done;
}

// 256 threads, thread 0 holding the highest bin: finds the thread at which the
// running count (from thread 0 on) reaches `need`.  Returns that thread's index
// (or -1 if the total stays below `need`), the count before it, the total, and
// that thread's own count.  `scratch` is LDS of 8 words.
__device__ __forceinline__ int block_threshold_scan(uint32_t mine, uint32_t need, uint32_t* scratch,
                                                    uint32_t& before_out, uint32_t& total_out,
                                                    uint32_t& count_out) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint32_t incl = mine;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == 63) scratch[wave] = incl;
  if (tid == 0) scratch[4] = 0xffffffffu;
  __syncthreads();
  uint32_t wave_base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (w < wave) wave_base += scratch[w];
    total += scratch[w];
  }
  const uint32_t before = wave_base + incl - mine;
  if (before < need && need <= before + mine) {
    scratch[4] = (uint32_t)tid;
    scratch[5] = before;
    scratch[6] = mine;
  }
  __syncthreads();
  const uint32_t who = scratch[4];
  before_out = scratch[5];
  count_out = scratch[6];
  total_out = total;
  __syncthreads();
  return who == 0xffffffffu ? -1 : (int)who;
}

// Votes-only launches: a phase ends with the memory idle while its statistics are on
// their way, and when a request takes the whole device no other phase streams meanwhile.
// The wavefronts that do not poll for the statistics touch the first keys of the
// workgroup that is going to take this one's place: `resident` workgroups further on in
// the grid, hence on the same XCD, whose L2 then holds what each of that workgroup's
// wavefronts asks for first.  One 4-byte load per 128-byte line; the values are only
// kept so that the loads are (the caller hands them to an empty asm at its end).
// Eight tokens per wavefront of the successor (64 KB per workgroup at eight KV heads, 2 MB
// per XCD): C5 layer 425 -> 420 us, C3 442 -> 438 us; 16 tokens bring less, 24 are slower
// than none (the L2 of an XCD holds 4 MB).
constexpr int kAheadTokens = 8;
constexpr int kAheadLoads = (4 * kAheadTokens * 16 + 191) / 192;  // per lane, at 16 lines per row
template <int HKV>
__device__ __forceinline__ void touch_successor_keys(const ScoreArgs& a, int wave, int lane,
                                                     uint32_t (&got)[kAheadLoads]) {
  constexpr uint32_t ROW_BYTES = HKV * kHeadDim * 2;
  constexpr int kLines = (int)ROW_BYTES / 128;
  constexpr int kItems = 4 * kAheadTokens * kLines;
  static_assert(kItems <= kAheadLoads * 192, "three wavefronts cover the lines");
#pragma unroll
  for (int i = 0; i < kAheadLoads; ++i) got[i] = 0u;
  const int g = (int)blockIdx.x + a.resident;
  if (a.resident <= 0 || g >= (int)gridDim.x) return;
  int phase = 0;
  while (phase + 1 < a.nphases && g >= a.phases[phase + 1].first_workgroup) ++phase;
  const VotePhase& ph = a.phases[phase];
  const int x = g - ph.first_workgroup;
  int req = 0;
  while (req + 1 < ph.requests && x >= ph.pack_first[req + 1]) ++req;
  const int b = ph.first + req;
  if (a.skip && a.skip[b]) return;
  const ReqGeom geo =
      request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
  const int block_lo = (x - ph.pack_first[req]) * ph.tokens_per_block;
  if (block_lo >= geo.n) return;
  const int per_wave = ph.tokens_per_block >> 2;
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;
#pragma unroll
  for (int i = 0; i < kAheadLoads; ++i) {
    const int item = (wave - 1) * 64 + lane + 192 * i;
    if (item < kItems) {
      const int t = item / kLines, line = item % kLines;
      const int tok = min(block_lo + (t / kAheadTokens) * per_wave + t % kAheadTokens, geo.n - 1);
      const int pos = a.n_init + tok;
      uint32_t slot = ((uint32_t)tab[pos >> a.page_shift] << a.page_shift) + (uint32_t)(pos & (a.page_size - 1));
      slot = slot < a.pool_rows ? slot : a.pool_rows - 1;
      got[i] = *(const uint32_t*)((const char*)a.k_pool + (size_t)slot * ROW_BYTES + line * 128);
    }
  }
}

template <int HKV, int G, bool OUT_BF16, int MODE>
__global__ __launch_bounds__(256, (G > 4 ? 1 : 2)) void score_kernel(ScoreArgs a) {
  extern __shared__ float stage[];  // tiled / fused: [tiles of the workgroup][tile_stride]
  constexpr bool TILED = MODE != kScoreDirect;
  constexpr bool FUSED = MODE == kScoreFused || MODE == kScorePacked;
  constexpr bool PACKED = MODE == kScorePacked;
  constexpr int TG = 8 / HKV;
  constexpr int UNITS = 8;
  constexpr int HALF = UNITS / 2;
  constexpr int NA = (G + 3) / 4;  // A operands (4 query heads each) per KV head
  constexpr int ITER = 16 * TG;    // tokens per iteration
  constexpr uint32_t ROW_BYTES = HKV * kHeadDim * 2;

  // This workgroup's request within the launch, and its chunk of that request.
  LaunchPart lp{a.tokens_per_block, a.batch_offset, 0, nullptr, (int)blockIdx.x, a.sync};
  int req = blockIdx.y, chunk = blockIdx.x;
  int req_chunks = (int)gridDim.x;  // chunks of this workgroup's request (the single launch: dealt)
  GridTeam team{0u, 0u};
  if (PACKED) {
    TS_MARK(0);
    // This workgroup's phase, and its request and chunk within the phase.
    int phase = 0;
    while (phase + 1 < a.nphases && (int)blockIdx.x >= a.phases[phase + 1].first_workgroup) ++phase;
    const VotePhase& ph = a.phases[phase];
    lp = LaunchPart{ph.tokens_per_block, ph.first, ph.requests, ph.pack_first,
                      (int)blockIdx.x - ph.first_workgroup, a.sync + (size_t)phase * kSyncWords};
    req = 0;
    while (req + 1 < lp.packed && lp.x >= lp.pack_first[req + 1]) ++req;
    chunk = lp.x - lp.pack_first[req];
  }
  if constexpr (FUSED && !PACKED) {
    __shared__ int deal_lds[8];
    TS_MARK(0);
    // The parts of the output that need no votes: request w % B by workgroup w / B of its share.
    {
      const int B = a.batch, w = (int)blockIdx.x, T = (int)gridDim.x;
      fixed_segments(a, a.batch_offset + w % B, w / B, (T - w % B + B - 1) / B);
    }
    const Deal deal = deal_workgroups(a, deal_lds);
    if (deal.req < 0) return;  // no chunk left for this workgroup
    lp.tokens_per_block = deal.tokens_per_block;
    req = deal.req;
    chunk = deal.chunk;
    req_chunks = deal.chunks;
    team = GridTeam{deal.team_size, deal.team_index};
  }
  const int b = req + lp.batch_offset;
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
  const int block_lo = chunk * lp.tokens_per_block;
  // (asked for here, long before it is used: the bin of the request's last selection)
  const int hint_word = (FUSED && !PACKED && a.hint) ? a.hint[b] : 0;
  if constexpr (PACKED) {
    __shared__ uint32_t team_lds[8];
    if (n <= 0) return;  // dense or served by the cache: nothing to select, not on the team
    if (block_lo >= n) return;  // no candidates here, and the team is made without it
    if (chunk == 0 && threadIdx.x == 0 &&
        (n + lp.tokens_per_block - 1) / lp.tokens_per_block > lp.pack_first[req + 1] - lp.pack_first[req])
      __hip_atomic_store(&lp.sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // length above its bound
    team = selecting_team<PACKED>(a, lp, team_lds, req, chunk);
  }
  if (block_lo >= n) return;  // (a dealt workgroup always has tokens)

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rg = lane >> 4;        // k-group of the operands, row group of the result
  const int t4 = (lane & 15) >> 2;  // token of a 4-token group / query of a 4-query group
  const int p = lane & 3;           // quarter of the head dimension
  const uint32_t lane_off = (uint32_t)(rg * 64 + p * 16);
  const int H = a.num_heads;
  // Fused: one spare row per tile keeps the four tiles a wavefront reads in the
  // vote phase on different LDS banks.
  const int tile_stride = FUSED ? 16 * H + 16 : 16 * H;
  const int32_t* tab = a.table + (int64_t)b * a.table_stride;

  // A operands: query 4*na + t4 of each KV head, same byte offsets as the keys.
  bf16x8_t qa[HKV][NA];
#pragma unroll
  for (int kvh = 0; kvh < HKV; ++kvh)
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      const int g = 4 * na + t4;
      const int h = head_of<HKV, G>(kvh, g < G ? g : 0, a.head_map);
      uint4 v;
      if (FUSED && !PACKED && a.q_raw != nullptr) {
        // The caller's un-rotated query: this lane's 8 dims and the 8 dims 64 further on (or
        // back), rotated as the rotation kernel does it.
        const bool lower = rg < 2;
        const uint32_t other_off = lower ? lane_off + 128u : lane_off - 128u;
        const char* qrow = (const char*)(a.q_raw + ((size_t)b * H + h) * kHeadDim);
        const uint4 own = *(const uint4*)(qrow + lane_off), other = *(const uint4*)(qrow + other_off);
        const float4 c0 = *(const float4*)((const char*)a.q_cos + 2 * lane_off);
        const float4 c1 = *(const float4*)((const char*)a.q_cos + 2 * lane_off + 16);
        const float4 s0 = *(const float4*)((const char*)a.q_sin + 2 * lane_off);
        const float4 s1 = *(const float4*)((const char*)a.q_sin + 2 * lane_off + 16);
        const uint32_t ow[4] = {own.x, own.y, own.z, own.w}, th[4] = {other.x, other.y, other.z, other.w};
        const float cs[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const float sn[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
        uint32_t r[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float lo = rotate_element(bf16_lo(ow[e]), bf16_lo(th[e]), cs[2 * e], sn[2 * e], lower);
          const float hi = rotate_element(bf16_hi(ow[e]), bf16_hi(th[e]), cs[2 * e + 1], sn[2 * e + 1], lower);
          r[e] = (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
        }
        v = make_uint4(r[0], r[1], r[2], r[3]);
      } else {
        v = *(const uint4*)((const char*)(a.qf + ((size_t)b * H + h) * kHeadDim) + lane_off);
      }
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

  const int per_wave = lp.tokens_per_block >> 2;
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
    const int tiles = (min(lp.tokens_per_block, n - block_lo) + 15) >> 4;
    float4* dst = (float4*)((float*)a.scores + ((size_t)b * a.score_stride + block_lo) * H);
    const float4* src = (const float4*)stage;
    for (int i = threadIdx.x; i < tiles * H * 4; i += 256) dst[i] = src[i];
  }
  if (a.partials == nullptr) return;

  // Per-workgroup (max, sum exp) of every head: 16 lanes of a row, then 4 waves.
  __shared__ float local_max[FUSED ? kMaxHeads : 1];  // by head slot
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
      float2* out = (float2*)a.partials + ((size_t)b * H + h) * a.nchunks + chunk;
      if (FUSED) {
        store_coherent(out, m, l);
        local_max[kvh * G + g] = m;
      } else {
        *out = make_float2(m, l);
      }
    }
  }

  if constexpr (FUSED) {
    __shared__ float s_rz[kMaxHeads];
    __shared__ uint32_t lh[kTopkBins];
    __shared__ uint32_t scratch[16];
    const int tid = threadIdx.x;
    static_assert(kBandSlots == 4, "a workgroup's candidates of a bin are one 16-byte piece");
    __shared__ uint32_t band_lds[kBandBins][kBandSlots];
    __shared__ uint32_t band_count[kBandBins + 1];  // per bin; [kBandBins]: tokens above the band
    for (int i = tid; i < kTopkBins; i += 256) lh[i] = 0u;
    if (tid < 16) scratch[tid] = 0u;
    if (tid < kBandBins * kBandSlots) band_lds[tid / kBandSlots][tid % kBandSlots] = 0u;
    if (tid <= kBandBins) band_count[tid] = 0u;
    TS_MARK(1);
    __syncthreads();  // scores, own maxima and the cleared histogram are in LDS for all
    TS_MARK(2);
    merge_request_stats<PACKED>(a, lp, team, lane, wave);
    TS_MARK(3);
    uint32_t ahead[kAheadLoads];
#pragma unroll
    for (int i = 0; i < kAheadLoads; ++i) ahead[i] = 0u;
    if constexpr (PACKED) {
      if (wave != 0) touch_successor_keys<HKV>(a, wave, lane, ahead);  // (wavefront 0 polls)
    }
    // While the merged statistics are on their way: the exponentials, relative to this
    // workgroup's own maxima; exp(s - max) / sum = exp(s - own max) * exp(own max - max) / sum.
    const ReqGeom geo =
        request_geometry(a.seq_lens, a.k_per_req, b, a.n_init, a.n_local, a.top_k, a.max_seq_len);
    const uint32_t k = (uint32_t)geo.k;
    const int count = min(lp.tokens_per_block, n - block_lo);
    uint32_t* ctr = a.counters + (size_t)b * kSelCounterWords;
    auto column = [&](int i) -> float* { return stage + (i >> 4) * tile_stride + (i & 15); };
    auto key_of = [&](int i) -> uint32_t { return vote_key(*column(i)); };
    for (int i = tid; i < count; i += 256) {
      float* sc = column(i);
#pragma unroll
      for (int s0 = 0; s0 < HKV * G; s0 += 8) {  // H = HKV * G head slots, 8 LDS reads in flight
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = s0 + j < HKV * G ? sc[(s0 + j) * 16] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < HKV * G) sc[(s0 + j) * 16] = __expf(x[j] - local_max[s0 + j]);
      }
    }
    if (tid < H) {  // H <= kMaxHeads < 256
      const int h = head_of<HKV, G>(tid / G, tid % G, a.head_map);
      const uint64_t* rep = (const uint64_t*)(a.stats + (size_t)(team.index % kSyncSlots) * a.stats_stride) +
                            (size_t)b * H + h;
      const uint64_t st = poll_nonzero<kStatsPollSleep>(rep, lp.sync, a.spin_ticks);
      const float mx = __uint_as_float((uint32_t)st), sum = __uint_as_float((uint32_t)(st >> 32));
      s_rz[tid] = st ? __expf(local_max[tid] - mx) / sum : 0.f;  // 0: the wait gave up
    }
    __syncthreads();
    TS_MARK(4);

    // Votes of this workgroup's tokens: fp32 sum over the head slots in slot order.
    // The vote replaces the first score of its token in LDS (only the thread that
    // owns a token reads its column).
    for (int i = tid; i < count; i += 256) {
      float* sc = column(i);
      float c = 0.f;
#pragma unroll
      for (int s0 = 0; s0 < HKV * G; s0 += 8) {
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = s0 + j < HKV * G ? sc[(s0 + j) * 16] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < HKV * G) c += x[j] * s_rz[s0 + j];
      }
      if (a.votes && a.pool_kernel <= 0) a.votes[(size_t)b * a.vote_stride + block_lo + i] = c;
      sc[0] = c;
    }
    TS_MARK(5);
    uint32_t round = 0;  // rendezvous passed so far
    if (a.pool_kernel > 0) {
      // Max-pool smoothing of the votes (tr.py:366-369): stride 1, padding (kernel-1)/2
      // with -inf, an even kernel makes the result one shorter.  The workgroups
      // exchange their votes through memory (one more rendezvous), gather the
      // kernel-1 neighbours on either side of their range into LDS (the histogram
      // array is still unused) and replace each vote by the maximum of its window.
      float* pv = a.pool_votes + (size_t)b * a.pool_stride;
      float* window = (float*)lh;  // [pad | own votes | kernel-1-pad]
      const int pad = (a.pool_kernel - 1) / 2;
      const int halo = a.pool_kernel - 1;
      for (int i = tid; i < count; i += 256) {
        const float c = *column(i);
        __hip_atomic_store((uint32_t*)&pv[block_lo + i], __float_as_uint(c), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        window[pad + i] = c;
      }
      grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
      for (int hx = tid; hx < halo; hx += 256) {
        const int t = hx < pad ? block_lo - pad + hx : block_lo + count + (hx - pad);
        const int at = hx < pad ? hx : count + hx;
        window[at] = (t >= 0 && t < n) ? __uint_as_float(load_coherent((const uint32_t*)&pv[t]))
                                       : -INFINITY;
      }
      __syncthreads();
      const int n_pooled = n + 2 * pad - a.pool_kernel + 1;
      for (int i = tid; i < count; i += 256) {
        float m = -INFINITY;  // past the pooled length: never selected (k < n)
        if (block_lo + i < n_pooled) {
          for (int w = 0; w < a.pool_kernel; ++w) m = fmaxf(m, window[i + w]);
          if (a.votes) a.votes[(size_t)b * a.vote_stride + block_lo + i] = m;
        }
        *column(i) = m;
      }
      __syncthreads();
      for (int i = tid; i < count + halo; i += 256) lh[i] = 0u;
      __syncthreads();
    }
    if (PACKED) {
      // The launch ends here: the votes are in memory, and their first histogram level
      // goes to the top-k workspace, where the kernels after this one pick it up.
      if (a.hist_ws) {
        for (int i = tid; i < count; i += 256) atomicAdd(&lh[key_bin0(key_of(i))], 1u);
        __syncthreads();
        uint32_t* hist0 = topk_ws(a.hist_ws, a.hist_ws_stride, b) + kTopkHist0;
        for (int i = tid; i < kTopkBins; i += 256)
          if (lh[i]) atomicAdd(&hist0[i], lh[i]);
      }
      if (chunk == 0 && tid == 0 && load_coherent(&lp.sync[0]) != 0u) {
        __hip_atomic_store(a.fault_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (a.fault_out)
          __hip_atomic_store(a.fault_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      }
#pragma unroll
      for (int i = 0; i < kAheadLoads; ++i) asm volatile("" ::"v"(ahead[i]));
      return;
    }
    // The physical slots of this thread's tokens, for the emission at the very end: the
    // table entries are asked for here, several rendezvous ahead, instead of in the
    // kernel's last microsecond with the stores waiting behind them.
    constexpr int kEmitAhead = 5;  // x 256 tokens: the largest workgroup (1056 tokens)
    uint32_t slot_ahead[kEmitAhead];
#pragma unroll
    for (int it = 0; it < kEmitAhead; ++it) {
      const int i = min(it * 256 + tid, count - 1);
      slot_ahead[it] = lookup_slot(tab, a.n_init + block_lo + i, a.page_size, a.page_shift, a.pool_rows);
    }
    // Local histogram: one LDS atomic per candidate (lanes that hit the same bin are
    // performed one after the other, which for 256 candidates is a few hundred cycles).
    // With a hint, also what the band around it needs: the candidates of each band bin go
    // to slots in LDS (published below), and the tokens above the band are counted.
    const int hint_bin = hint_word - 1;
    const bool banded = hint_bin >= 0 && hint_bin < kTopkBins && lp.tokens_per_block <= kBandMaxTokens &&
                        req_chunks <= kSelMaxChunks / 2;
    const int band_lo = hint_bin - kBandBelow;  // (bins outside [0, kTopkBins) hold nothing)
    uint32_t over_band = 0;  // this thread's tokens above the band
    uint32_t top = 0;        // this thread's highest bin
    for (int base = 0; base < count; base += 256) {
      const bool have = base + tid < count;
      const uint32_t key = have ? key_of(base + tid) : 0u;
      const uint32_t bin = have ? key_bin0(key) : 0u;
      if (have) atomicAdd(&lh[bin], 1u);
      top = max(top, bin);
      if (banded) {
        const int d = (int)bin - band_lo;
        if (have && d >= 0 && d < kBandBins) {
          const uint32_t at = atomicAdd(&band_count[d], 1u);
          if (at < (uint32_t)kBandSlots)
            band_lds[d][at] = 0x80000000u | ((key & 0x1fffffu) << 10) | (uint32_t)(base + tid);
        }
        over_band += (have && d >= kBandBins) ? 1u : 0u;
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, off));
    if (lane == 0) atomicMax(&scratch[8], top);
    if (banded) {
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) over_band += __shfl_xor(over_band, off);
      if (lane == 0 && over_band) atomicAdd(&band_count[kBandBins], over_band);
    }
    __syncthreads();

    TS_MARK(6);
    // First level: top 11 key bits.  The workgroups add their local histograms to one
    // of the copies and note the highest occupied bin; afterwards each searches
    // downwards from that bin, 256 bins at a time (one is enough unless the votes
    // span more than 64 binades).
    uint32_t* hist0 = ctr + kSelHist0 + (chunk % kSelHistCopies) * kTopkBins;
    {
      // Two adjacent bins per 64-bit add (their counts cannot carry into each other):
      // half as many read-modify-writes on the few hot lines.
      uint64_t done = 0;  // old values: waited for once, after all are on their way
#pragma unroll
      for (int j = 0; j < kTopkBins / 512; ++j) {
        const int i = 2 * (tid + 256 * j);
        const uint64_t pair = (uint64_t)lh[i] | ((uint64_t)lh[i + 1] << 32);
        if (pair)
          done += __hip_atomic_fetch_add((uint64_t*)&hist0[i], pair, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
      }
      if (tid == 0)
        done += fetch_max_coherent(&ctr[kSelMaxBin + (chunk % kSelHistCopies) * 32], scratch[8]);
      if (banded && wave == 1) {
        // The band.  Lane l holds the count of band bin l (lane kBandBins: of the bins above
        // the band); the tokens above bin l are the sum over the lanes after it.
        uint4* slots = a.band_slots + (size_t)b * kBandBins * kSelMaxChunks;
        uint32_t* above = a.band_above + (size_t)b * kBandBins * kSelMaxChunks;
        const uint32_t here = lane <= kBandBins ? band_count[lane] : 0u;
        uint32_t run = here;  // becomes the sum over lanes l .. l + 15
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
          const uint32_t up = (uint32_t)__shfl_down((int)run, off);
          run += lane + off < 64 ? up : 0u;
        }
        static_assert(kBandBins + 1 <= 16, "the sum spans the band");
        if (lane < kBandBins) {
          done += __hip_atomic_exchange(&above[(size_t)lane * kSelMaxChunks + chunk], ((run - here) << 16) | here,
                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          // (the candidates: the first 8-byte half of the piece, the second only if used)
          uint64_t* piece = (uint64_t*)&slots[(size_t)lane * kSelMaxChunks + chunk];
          if (here >= 1)
            done += __hip_atomic_exchange(piece, (uint64_t)band_lds[lane][0] | ((uint64_t)band_lds[lane][1] << 32),
                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          if (here >= 3)
            done += __hip_atomic_exchange(piece + 1, (uint64_t)band_lds[lane][2] | ((uint64_t)band_lds[lane][3] << 32),
                                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (lane <= kBandBins && here)
          done += fetch_add_coherent(&ctr[kSelBandHist + (chunk % kBandHistCopies) * 32 + lane], here);
      }
      await(done);
    }
    TS_MARK(7);
    grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
    TS_MARK(8);
    uint32_t t0 = 0, above0 = 0, in_bin0 = 0;
    // With a hint: the band's small histogram, the flags, the counts of the workgroups before
    // this one and every workgroup's slots for the bin the hint names are requested
    // together (the bin is a guess: the threshold bin is known after the search, and
    // another bin of the band costs one more round of loads).
    constexpr int kBandLoads = kSelMaxChunks / 2 / 256;  // (512 chunks at most)
    uint32_t band_word[kBandLoads];
    uint4 band_piece[kBandLoads];
    auto load_band = [&](int d) {
      const uint32_t* above = a.band_above + ((size_t)b * kBandBins + d) * kSelMaxChunks;
      const uint4* slots = a.band_slots + ((size_t)b * kBandBins + d) * kSelMaxChunks;
#pragma unroll
      for (int r = 0; r < kBandLoads; ++r) {
        const int at = tid + 256 * r;
        band_word[r] = 0u;
        band_piece[r] = make_uint4(0u, 0u, 0u, 0u);
        if (at < req_chunks) {
          band_word[r] = load_coherent(&above[at]);
          const uint64_t lo = __hip_atomic_load((const uint64_t*)&slots[at], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          const uint64_t hi = __hip_atomic_load((const uint64_t*)&slots[at] + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          band_piece[r] = make_uint4((uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32));
        }
      }
    };
    bool found = false;     // the threshold bin is known
    bool from_band = false; // and the band's slots hold its candidates
    if (banded) {
      uint32_t* band_hist = lh + 1960;   // [kBandBins + 1] (the histogram array is free again)
      if (tid <= kBandBins) band_hist[tid] = 0u;
      if (tid == 32) lh[2000] = 0u;      // a workgroup with more candidates in the bin than slots
      __syncthreads();
      constexpr int kWords = kBandHistCopies * (kBandBins + 1);
      constexpr int kPerThread = (kWords + 255) / 256;
      uint32_t part[kPerThread];
#pragma unroll
      for (int r = 0; r < kPerThread; ++r) {
        const int word = tid + 256 * r;
        part[r] = word < kWords
                      ? load_coherent(&ctr[kSelBandHist + (word / (kBandBins + 1)) * 32 + word % (kBandBins + 1)])
                      : 0u;
      }
      load_band(kBandBelow);
#pragma unroll
      for (int r = 0; r < kPerThread; ++r)
        if (part[r]) atomicAdd(&band_hist[(tid + 256 * r) % (kBandBins + 1)], part[r]);
      __syncthreads();
      // Downwards from the bins above the band: the bin in which the count reaches k.
      uint32_t run = band_hist[kBandBins];
      int d0 = -1;
      if (run < k) {
        for (int d = kBandBins - 1; d >= 0; --d) {
          const uint32_t here = band_hist[d];
          if (run + here >= k) {
            d0 = d;
            in_bin0 = here;
            break;
          }
          run += here;
        }
      }
      if (d0 >= 0 && band_lo + d0 >= 0) {
        found = true;
        t0 = (uint32_t)(band_lo + d0);
        above0 = run;
        if (in_bin0 <= (uint32_t)kSelListCap) {
          if (d0 != kBandBelow) load_band(d0);
          bool fits = true;
#pragma unroll
          for (int r = 0; r < kBandLoads; ++r) fits = fits && (band_word[r] & 0xffffu) <= (uint32_t)kBandSlots;
          if (!fits) lh[2000] = 1u;
          __syncthreads();
          from_band = lh[2000] == 0u;
        }
      }
      __syncthreads();
    }
    if (!found) {
    // The search starts at the highest occupied bin of the request.  Together with the
    // words that hold it, the 128 bins below a guess (a little above this workgroup's
    // own highest bin) are fetched; the guess serves if no bin above it is occupied.
    constexpr int kWindow = 128;  // bins per step: two threads per bin, half the copies each
    const int guess = min((int)scratch[8] + 32, kTopkBins - 1);
    auto bins_below = [&](int top) {
      const int bin = top - (tid >> 1);
      const int first = (tid & 1) * (kSelHistCopies / 2);
      uint32_t part[kSelHistCopies / 2];
#pragma unroll
      for (int c = 0; c < kSelHistCopies / 2; ++c)
        part[c] = bin >= 0 ? load_coherent(&ctr[kSelHist0 + (first + c) * kTopkBins + bin]) : 0u;
      uint32_t sum = 0;
#pragma unroll
      for (int c = 0; c < kSelHistCopies / 2; ++c) sum += part[c];
      sum += (uint32_t)__shfl_xor((int)sum, 1);
      return (tid & 1) ? 0u : sum;  // the even thread of a pair stands for the bin
    };
    uint32_t mine = bins_below(guess);
    int top = guess;
    {
      uint32_t m = tid < kSelHistCopies ? load_coherent(&ctr[kSelMaxBin + tid * 32]) : 0u;
#pragma unroll
      for (int off = kSelHistCopies / 2; off >= 1; off >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, off));
      __syncthreads();  // every thread has read this workgroup's own highest bin
      if (tid == 0) scratch[8] = m;
      __syncthreads();
      if ((int)scratch[8] > guess) {
        top = (int)scratch[8];
        mine = bins_below(top);
      }
    }
    for (;;) {
      uint32_t before, total, in_bin;
      const int who = block_threshold_scan(mine, k - above0, scratch, before, total, in_bin);
      if (who >= 0) {
        t0 = (uint32_t)(top - (who >> 1));
        above0 += before;
        in_bin0 = in_bin;
        break;
      }
      above0 += total;
      top -= kWindow;
      if (top < 0) break;
      mine = bins_below(top);
    }
    }

    TS_MARK(9);
    // What is left: `need` of the `in_bin` candidates whose key >> shift equals `prefix`.
    // As soon as they are few enough, they go to a short list that every workgroup
    // ranks on its own (the usual case: heavy-tailed votes leave a hundred candidates
    // in the threshold bin of the first level); otherwise the next histogram level.
    uint32_t need = k - above0, in_bin = in_bin0, prefix = t0;
    int shift = 21;
    if (in_bin > (uint32_t)kSelListCap) {
      // Second level: next 11 bits of the candidates inside bin t0.
      uint32_t done = 0;
      for (int base = 0; base < count; base += 256) {
        const uint32_t key = base + tid < count ? key_of(base + tid) : 0u;
        done += wave_histogram_add(ctr + kSelHist1 + (chunk % kSelHist1Copies) * kTopkBins,
                                   base + tid < count && key_bin0(key) == t0, key_bin1(key), lane);
      }
      await(done);
      grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
      {
        uint32_t h[kTopkBins / 256];
#pragma unroll
        for (int j = 0; j < kTopkBins / 256; ++j) {
          uint32_t part[kSelHist1Copies];
#pragma unroll
          for (int c = 0; c < kSelHist1Copies; ++c)
            part[c] = load_coherent(&ctr[kSelHist1 + c * kTopkBins + tid + 256 * j]);
          h[j] = 0u;
#pragma unroll
          for (int c = 0; c < kSelHist1Copies; ++c) h[j] += part[c];
        }
#pragma unroll
        for (int j = 0; j < kTopkBins / 256; ++j) lh[tid + 256 * j] = h[j];
      }
      __syncthreads();
      uint32_t t1, above1;
      find_threshold_bin<kTopkBins>(lh, need, scratch, t1, above1);
      need -= above1;
      in_bin = lh[t1];
      prefix = (t0 << 11) | t1;
      shift = 10;
      __syncthreads();
    }

    uint2* counts = a.block_counts + (size_t)b * kSelMaxChunks;
    const bool listed = in_bin <= (uint32_t)kSelListCap;
    uint32_t kth, need_eq = 0, pos_thr = 0;
    if (tid < 8) scratch[8 + tid] = 0u;
    __syncthreads();
    // With a hint whose band holds the threshold bin, everything the ranking needs was
    // published before the first rendezvous: no list round.  The test was the same for every
    // workgroup of the request (the band's histogram, the flags), so all take the same way.
    bool has = false;
    uint2 e = make_uint2(0u, 0u);
    if (from_band) {
      uint2* entries_lds = (uint2*)(lh + 1024);  // [kSelListCap]
      uint32_t band_sure = 0;  // tokens above the bin in the workgroups before this one
#pragma unroll
      for (int r = 0; r < kBandLoads; ++r) {
        const uint32_t packed[4] = {band_piece[r].x, band_piece[r].y, band_piece[r].z, band_piece[r].w};
        const uint32_t from = (uint32_t)(tid + 256 * r) * (uint32_t)lp.tokens_per_block;  // that workgroup's first token
        const uint32_t have = band_word[r] & 0xffffu;  // (zero where the load was skipped)
        if (tid + 256 * r < chunk) band_sure += band_word[r] >> 16;
#pragma unroll
        for (int h2 = 0; h2 < 4; ++h2)
          if ((uint32_t)h2 < have) {
            const uint32_t at = atomicAdd(&scratch[15], 1u);
            if (at < (uint32_t)kSelListCap)
              entries_lds[at] = make_uint2((t0 << 21) | ((packed[h2] >> 10) & 0x1fffffu), from + (packed[h2] & 1023u));
          }
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) band_sure += __shfl_xor(band_sure, off);
      if (lane == 0) atomicAdd(&scratch[10], band_sure);
      __syncthreads();
      // (every candidate of the bin is in a slot: the count is that of the histogram)
      if (scratch[15] != in_bin && tid == 0)
        __hip_atomic_store(&lp.sync[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      has = (uint32_t)tid < min(scratch[15], (uint32_t)kSelListCap);
      if (has) e = entries_lds[tid];
      __syncthreads();
      TS_MARK(10);
    } else if (listed) {
      // Last round, short form: the candidates of the threshold bin are appended to
      // the list (in kSelListParts parts with a counter each, a wavefront reserving
      // its entries with one add), and every workgroup publishes how many of its
      // tokens lie above the bin.
      uint2* list = a.short_list + (size_t)b * kSelListParts * kSelListCap;
      const int part = chunk % kSelListParts;
      const uint64_t below_mask = (1ull << lane) - 1ull;
      uint32_t above = 0;
      for (int base = 0; base < count; base += 256) {
        const int i = base + tid;
        const uint32_t key = i < count ? key_of(i) : 0u;
        const uint32_t top = key >> shift;
        above += (i < count && top > prefix) ? 1u : 0u;
        const bool match = i < count && top == prefix;
        const uint64_t mm = __ballot(match);
        if (mm) {
          const int leader = __ffsll((unsigned long long)mm) - 1;
          uint32_t slot = 0;
          if (lane == leader)
            slot = fetch_add_coherent(&ctr[kSelListCount + part * 32], (uint32_t)__popcll(mm));
          slot = (uint32_t)__shfl((int)slot, leader) + (uint32_t)__popcll(mm & below_mask);
          if (match && slot < (uint32_t)kSelListCap)
            store_coherent(&list[part * kSelListCap + slot], key, (uint32_t)(block_lo + i));
        }
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) above += __shfl_xor(above, off);
      if (lane == 0) atomicAdd(&scratch[8], above);
      __syncthreads();
      if (tid == 0) store_coherent(&counts[chunk], scratch[8], 0u);
      TS_MARK(10);
      grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
      TS_MARK(11);

      // Every workgroup ranks the list on its own, one entry per thread, in the order
      // (key descending, position ascending) packed into one 64-bit word.  The fill
      // counters, the entries (thread t guesses entry t / parts of part t % parts,
      // which is right unless a part holds more than 256 / parts) and the counts of
      // the workgroups before this one are fetched together.
      constexpr uint32_t kPerPart = kSelListCap / kSelListParts;
      const uint32_t fill =
          tid < kSelListParts ? load_coherent(&ctr[kSelListCount + tid * 32]) : 0u;
      e = load_coherent(&list[(tid % kSelListParts) * kSelListCap + tid / kSelListParts]);
      {
        uint32_t sure = 0;
        for (int j = tid; j < chunk; j += 256) sure += load_coherent(&counts[j]).x;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) sure += __shfl_xor(sure, off);
        if (lane == 0) atomicAdd(&scratch[10], sure);
      }
      if (tid < kSelListParts) scratch[tid] = min(fill, (uint32_t)kSelListCap);
      __syncthreads();
      uint32_t entries = 0, longest = 0;
#pragma unroll
      for (int p = 0; p < kSelListParts; ++p) {
        entries += scratch[p];
        longest = max(longest, scratch[p]);
      }
      if (longest <= kPerPart) {
        has = (uint32_t)tid / kSelListParts < scratch[tid % kSelListParts];
      } else {  // uneven parts: entry t of the concatenation
        uint32_t at = (uint32_t)tid, from = 0;
        has = false;
#pragma unroll
        for (int p = 0; p < kSelListParts; ++p) {
          if (!has && at < scratch[p]) {
            has = true;
            from = (uint32_t)p;
          } else if (!has) {
            at -= scratch[p];
          }
        }
        has = has && (uint32_t)tid < min(entries, (uint32_t)kSelListCap);
        if (has) e = load_coherent(&list[from * kSelListCap + at]);
      }
    }
    if (listed) {
      const uint64_t mine = has ? ((uint64_t)e.x << 32) | (uint64_t)(0xffffffffu - e.y) : 0ull;
      const uint32_t my_pos = e.y;
      // The need-th largest entry: one more histogram level, over the next 8 key bits
      // and in LDS, leaves the entries of one digit, which rank themselves against
      // each other (ranking all entries against all would cost 64 K comparisons).
      uint32_t* digits = lh;                    // [256]
      uint64_t* peers = (uint64_t*)(lh + 256);  // [kSelListCap] entries of the threshold digit
      const uint32_t digit = (e.x >> (shift - 8)) & 255u;
      digits[tid] = 0u;
      __syncthreads();
      if (has) atomicAdd(&digits[digit], 1u);
      __syncthreads();
      uint32_t above_digit, all_digits, in_digit;
      const int down = block_threshold_scan(digits[255 - tid], need, scratch, above_digit,
                                            all_digits, in_digit);
      const uint32_t threshold_digit = 255u - (uint32_t)down;  // down >= 0: the bin holds the k-th
      const bool peer = has && digit == threshold_digit;
      if (peer) peers[atomicAdd(&scratch[14], 1u)] = mine;
      __syncthreads();
      uint32_t rank = 0;
      if (peer)
        for (uint32_t u = 0; u < in_digit; ++u) rank += peers[u] > mine ? 1u : 0u;
      const uint32_t need_here = need - above_digit;
      const bool taken = has && (digit > threshold_digit || (peer && rank < need_here));
      if (peer && rank + 1 == need_here) {  // the k-th of the request
        scratch[9] = e.x;
        scratch[12] = my_pos;
      }
      const uint64_t lower = __ballot(taken && my_pos < (uint32_t)block_lo);
      if (lane == 0 && lower) atomicAdd(&scratch[13], (uint32_t)__popcll(lower));
      __syncthreads();
      kth = scratch[9];
      pos_thr = scratch[12];
      TS_MARK(12);
    } else {
      // Third level: last 10 bits of the candidates inside (t0, t1).
      const uint32_t t1 = prefix & 2047u;
      {
        uint32_t done = 0;
        for (int base = 0; base < count; base += 256) {
          const uint32_t key = base + tid < count ? key_of(base + tid) : 0u;
          done += wave_histogram_add(
              ctr + kSelHist2, base + tid < count && key_bin0(key) == t0 && key_bin1(key) == t1,
              key_bin2(key), lane);
        }
        await(done);
      }
      grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
      {
        uint32_t h[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) h[j] = load_coherent(&ctr[kSelHist2 + tid + 256 * j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) lh[tid + 256 * j] = h[j];
      }
      __syncthreads();
      uint32_t t2, above2;
      find_threshold_bin<1024>(lh, need, scratch, t2, above2);
      need_eq = need - above2;  // ties at the k-th key still to take
      kth = (t0 << 21) | (t1 << 10) | t2;

      // Count step: every workgroup publishes how many of its tokens lie above the k-th
      // key and how many tie with it; ties are taken lowest position first, so the
      // counts of the workgroups before this one fix where its output starts and
      // how many of its ties still fit.
      uint32_t sure = 0, tie = 0;
      for (int i = tid; i < count; i += 256) {
        const uint32_t key = key_of(i);
        sure += key > kth ? 1u : 0u;
        tie += key == kth ? 1u : 0u;
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        sure += __shfl_xor(sure, off);
        tie += __shfl_xor(tie, off);
      }
      if (lane == 0) {
        atomicAdd(&scratch[8], sure);
        atomicAdd(&scratch[9], tie);
      }
      __syncthreads();
      if (tid == 0) store_coherent(&counts[chunk], scratch[8], scratch[9]);
      grid_arrive(lp.sync, ++round, a.spin_ticks, team.size, team.index);
    }
    // The requests of a batch may need different numbers of rounds, and the rendezvous
    // spans them all: whoever is through counts itself in for the rounds it skipped.
    if (team.size != (uint32_t)req_chunks) {  // other requests select in this launch as well
      const uint32_t rounds = kSelectRounds + (a.pool_kernel > 0 ? 1u : 0u);
      grid_arrive_rest(lp.sync, round + 1, rounds, team.size, team.index);
      round = rounds;
    }
    if (!listed) {
      // Counts of the workgroups before this one.
      uint32_t sure = 0, tie = 0;
      for (int j = tid; j < chunk; j += 256) {
        const uint2 v = load_coherent(&counts[j]);
        sure += v.x;
        tie += v.y;
      }
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) {
        sure += __shfl_xor(sure, off);
        tie += __shfl_xor(tie, off);
      }
      if (lane == 0) {
        atomicAdd(&scratch[10], sure);
        atomicAdd(&scratch[11], tie);
      }
    }
    __syncthreads();
    TS_MARK(13);
    uint32_t tie_run = scratch[11];  // ties at lower positions
    // selected at lower positions
    uint32_t out_run = scratch[10] + (listed ? scratch[13] : min(tie_run, need_eq));
    __syncthreads();

    // Emission in position order.
    const int32_t* tab_b = a.table + (int64_t)b * a.table_stride;
    int32_t* sel = a.sel + (int64_t)b * a.sel_stride;
    int32_t* sel_pos = a.sel_pos + (int64_t)b * a.sel_stride;
    int32_t* cache_out = a.topk_cache ? a.topk_cache + (int64_t)b * a.top_k : nullptr;
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll 1
    for (int base = 0, it = 0; base < count; base += 256, ++it) {
      const int i = base + tid;
      const uint32_t key = i < count ? key_of(i) : 0u;
      const bool tie = i < count && key == kth;
      // The per-wavefront counts of an iteration go to one of two sets of words in turn: a
      // set is written again two iterations later, after a barrier that every wavefront
      // reaches only once it has read the set, so no barrier closes an iteration.
      uint32_t* counts_lds = scratch + (it & 1) * 8;
      uint32_t tie_rank = 0, tie_total = 0;
      if (!listed) {  // (with the short list a tie is taken by its position: no ranks needed)
        const uint64_t tie_mask = __ballot(tie);
        if (lane == 0) counts_lds[wave] = (uint32_t)__popcll(tie_mask);
        __syncthreads();
        tie_rank = tie_run + (uint32_t)__popcll(tie_mask & below);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          if (w < wave) tie_rank += counts_lds[w];
          tie_total += counts_lds[w];
        }
      }
      // A tie is taken if it is among the first need_eq in position order; with the
      // short list that is: not beyond the position of the k-th entry.
      const bool tie_taken = listed ? (uint32_t)(block_lo + i) <= pos_thr : tie_rank < need_eq;
      const bool chosen = i < count && (key > kth || (tie && tie_taken));
      const uint64_t chosen_mask = __ballot(chosen);
      if (lane == 0) counts_lds[4 + wave] = (uint32_t)__popcll(chosen_mask);
      __syncthreads();
      uint32_t rank = out_run + (uint32_t)__popcll(chosen_mask & below);
      uint32_t chosen_total = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        if (w < wave) rank += counts_lds[4 + w];
        chosen_total += counts_lds[4 + w];
      }
      if (chosen && rank < k) {
        const int pos = a.n_init + block_lo + i;
        sel_pos[a.n_init + rank] = pos;
        uint32_t slot = slot_ahead[0];
#pragma unroll
        for (int x = 1; x < kEmitAhead; ++x) slot = it == x ? slot_ahead[x] : slot;
        if (it >= kEmitAhead) slot = lookup_slot(tab_b, pos, a.page_size, a.page_shift, a.pool_rows);
        sel[a.n_init + rank] = (int32_t)slot;
        if (cache_out) cache_out[rank] = pos;
      }
      tie_run += tie_total;
      out_run += chosen_total;
    }
    TS_MARK(14);
    // A grid-wide wait of this launch gave up (the workgroups were not all resident
    // within the bound): what was selected is not valid.  The first workgroup of every
    // selecting request says so in place of the length, and in the caller's word.
    if (chunk == 0 && tid == 0) {
      const bool gave_up = load_coherent(&lp.sync[0]) != 0u;
      a.sel_len[b] = gave_up ? -1 : a.n_init + (int)k + a.n_local;
      if (a.hint && !gave_up) a.hint[b] = (int)t0 + 1;  // where the next step's band is going to lie
      if (gave_up && a.fault_out)
        __hip_atomic_store(a.fault_out, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
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
  TS_SCORE_CASE(HKV_, 1) TS_SCORE_CASE(HKV_, 2) TS_SCORE_CASE(HKV_, 3) TS_SCORE_CASE(HKV_, 4) \
      TS_SCORE_CASE(HKV_, 5) TS_SCORE_CASE(HKV_, 6) TS_SCORE_CASE(HKV_, 7) TS_SCORE_CASE(HKV_, 8)
  TS_SCORE_ROW(1)
  TS_SCORE_ROW(2)
  TS_SCORE_ROW(4)
  TS_SCORE_ROW(8)
#undef TS_SCORE_ROW
#undef TS_SCORE_CASE
  return fail(TS_ESHAPE, "unsupported head shape: num_kv_heads=%d group=%d", hkv, group);
}

// The fused kernel of a head shape (its packed votes-only form), or NULL.
static const void* fused_kernel_of(int hkv, int group, bool packed = false) {
#define TS_SCORE_CASE(HKV_, G_)                                                        \
  if (hkv == HKV_ && group == G_)                                                      \
    return packed ? (const void*)&score_kernel<HKV_, G_, false, kScorePacked>          \
                  : (const void*)&score_kernel<HKV_, G_, false, kScoreFused>;
#define TS_SCORE_ROW(HKV_) \
  TS_SCORE_CASE(HKV_, 1) TS_SCORE_CASE(HKV_, 2) TS_SCORE_CASE(HKV_, 3) TS_SCORE_CASE(HKV_, 4) \
      TS_SCORE_CASE(HKV_, 5) TS_SCORE_CASE(HKV_, 6) TS_SCORE_CASE(HKV_, 7) TS_SCORE_CASE(HKV_, 8)
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

// Dynamic LDS the fused form may use.  With the 10 KB of static arrays two workgroups
// of 68 KB fit the 160 KB of a CU; a workgroup that asks for more than half of a CU's LDS
// (up to 140 KB) has the CU to itself.  Which of the two a launch gets is decided by its
// planner (fused_tokens_per_block, plan_vote_launches).
constexpr size_t kFusedStageBytes = 68 * 1024;
constexpr size_t kFusedLargeStageBytes = 140 * 1024;
constexpr size_t kFusedLargeFloorBytes = 76 * 1024;  // more than half a CU's LDS: one workgroup per CU
static size_t fused_stage_bytes(bool large) { return large ? kFusedLargeStageBytes : kFusedStageBytes; }

// The one process-wide switch of the library (ts_set_fused_select).
static std::atomic<int> g_fused_select{1};

int set_fused_select(int enable) { return g_fused_select.exchange(enable ? 1 : 0); }

static thread_local bool g_separate_call = false;
bool fused_kernels_enabled() { return g_fused_select.load() != 0 && !g_separate_call; }
SeparateKernelsScope::SeparateKernelsScope(bool on) : was(g_separate_call) {
  if (on) g_separate_call = true;
}
SeparateKernelsScope::~SeparateKernelsScope() { g_separate_call = was; }

// Workgroups of the fused kernel that the current device keeps resident at once (0: the
// shape has no fused kernel, or the runtime refused); depends on the kernel only.
static int fused_capacity(const ts_config* cfg, bool packed, bool large) {
  const void* fn = fused_kernel_of(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads, packed);
  if (!fn) return 0;
  struct Entry { const void* fn; int device; bool large; int capacity; };
  static thread_local Entry memo[16] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  int capacity = 0;
  for (const Entry& e : memo)
    if (e.fn == fn && e.device == device && e.large == large) capacity = e.capacity;
  if (capacity == 0) {
    int per_cu = 0, cus = 0;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)kFusedLargeStageBytes) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, 256, fused_stage_bytes(large)) !=
            hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    capacity = per_cu * cus;
    if (capacity <= 0) return 0;
    static thread_local int next = 0;
    memo[next++ % 16] = Entry{fn, device, large, capacity};
  }
  return capacity;
}

// With max-pooling a workgroup gathers its votes and kernel - 1 neighbours into the LDS
// array of the histogram (kTopkBins words): the most tokens a workgroup may take then.
static int pooling_tokens_cap(const ts_config* cfg) {
  if (cfg->pool_kernel <= 0) return 1 << 30;
  return (kTopkBins - (cfg->pool_kernel - 1)) / 64 * 64;
}

// Tokens per workgroup of ts_select for a batch, 0 when the shape is not served; *large:
// whether the workgroups have a CU to themselves; *most_blocks: the most workgroups per
// request of any plan this shape may get (what has to be cleared for it).
// One workgroup per CU wherever the batch fits that way with no more LDS than a small
// workgroup has (C2 64.2 -> 61.9 us; 1.7-2.9 us at every length from 8K on for one request,
// 1-2 us for 2 x 64K and 4 x 32K): below 256 workgroups the dispatcher otherwise doubles
// them up on some CUs while others idle, above that half as many workgroups stream as
// fast and hand over less.  Batches that need more LDS per CU than that run as well or
// better on two workgroups per CU (2 x 128K the same, 4 x 64K and 8 x 32K 1-2 us better),
// unless requests may be skipped (selection cache): the workgroups are dealt over the
// requests that select, a step rarely has all of them, and the large workgroups then
// hold fewer tokens than they could (C4: 89.0 -> 87.4 us per step).
int fused_tokens_per_block(const ts_config* cfg, int batch, int max_seq_len, bool ignore_switch,
                           bool* large_out, bool may_skip, int* most_blocks_out) {
  if (large_out) *large_out = false;
  if (most_blocks_out) *most_blocks_out = 0;
  // Max-pool windows beyond 256 would not fit the LDS the neighbours are gathered into.
  if ((!ignore_switch && !fused_kernels_enabled()) || cfg->num_heads > kMaxHeads || cfg->pool_kernel > 256)
    return 0;
  const int max_n = max_seq_len - cfg->n_init - cfg->n_local;
  if (max_n <= 0) return 0;
  auto plan = [&](bool large) {
    const int capacity = fused_capacity(cfg, false, large);
    if (capacity <= 0) return 0;
    int tpb = score_tokens_per_block((int64_t)batch * max_seq_len, cfg->num_heads);
    while ((int64_t)ceil_div(max_n, tpb) * batch > capacity) tpb += 64;
    if (fused_lds_bytes(tpb, cfg->num_heads) > fused_stage_bytes(large) || tpb > pooling_tokens_cap(cfg))
      return 0;
    if (ceil_div(max_seq_len, tpb) > kSelMaxChunks) return 0;  // what the workspace is laid out for
    return tpb;
  };
  const int tpb_small = plan(false), tpb_large = plan(true);
  // (the workgroups of a launch are dealt over the requests that select: one request may
  // get them all)
  if (most_blocks_out)
    *most_blocks_out = std::min<int>(
        kSelMaxChunks, batch * std::max(tpb_small > 0 ? (int)ceil_div(max_n, tpb_small) : 0,
                                        tpb_large > 0 ? (int)ceil_div(max_n, tpb_large) : 0));
  const bool roomy = tpb_large > 0 && fused_lds_bytes(tpb_large, cfg->num_heads) <= kFusedStageBytes;
  if (roomy || tpb_small == 0 || (may_skip && batch >= 2 && tpb_large > 0)) {
    if (large_out) *large_out = tpb_large > 0;
    return tpb_large;
  }
  return tpb_small;
}

SelectWorkspace select_workspace(const ts_config* cfg, int batch, int max_seq_len, bool ignore_switch,
                                 bool may_skip) {
  SelectWorkspace w{};
  // The layout depends on the batch, the head count and (for the pooled votes) the
  // length, not on how the candidates are dealt out, and is the same whether or not
  // this shape is served: a workspace sized for the longest context serves every
  // shorter one.
  bool large = false;
  w.tokens_per_block =
      fused_tokens_per_block(cfg, batch, max_seq_len, ignore_switch, &large, may_skip, &w.clear_chunks);
  w.lds_bytes = w.tokens_per_block > 0
                    ? std::max(fused_lds_bytes(w.tokens_per_block, cfg->num_heads),
                               large ? kFusedLargeFloorBytes : (size_t)0)
                    : 0;
  const int max_n = std::max(max_seq_len - cfg->n_init - cfg->n_local, 0);
  w.blocks_per_req = w.tokens_per_block > 0 ? (int)ceil_div(max_n, w.tokens_per_block) : 0;
  const size_t B = (size_t)batch, H = (size_t)cfg->num_heads;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    const size_t at = off;
    off += align_up(bytes, 256);
    return at;
  };
  w.partials = take(B * H * (size_t)kSelMaxChunks * 2 * sizeof(float));
  // The counters and, right behind them, the replicas of the statistics are cleared
  // together before every launch.
  w.counters = take(B * kSelCounterWords * 4);
  w.stats_stride = (int64_t)align_up(B * H * 2, 1024);
  w.stats = take((size_t)kSyncSlots * w.stats_stride * sizeof(float));
  w.block_counts = take(B * (size_t)kSelMaxChunks * sizeof(uint2));
  w.short_list = take(B * kSelListParts * kSelListCap * sizeof(uint2));
  w.band_above = take(B * kBandBins * (size_t)kSelMaxChunks * sizeof(uint32_t));
  w.band_slots = take(B * kBandBins * (size_t)kSelMaxChunks * sizeof(uint4));
  w.pool_stride = (int64_t)align_up((size_t)std::max(max_n, 1), 64);
  w.pool_votes = take(cfg->pool_kernel > 0 ? B * (size_t)w.pool_stride * sizeof(float) : 0);
  w.sync = take(B * kSyncWords * 4);  // one rendezvous area per launch of a batch served in groups
  w.total = off;
  return w;
}

// One phase of the votes-only form: requests [first, first + requests), `workgroups` in
// all, `table_chunks` an upper bound of the chunks of any of its requests.
struct VoteLaunch {
  int first, requests, tokens_per_block, workgroups, table_chunks;
};
// The phases of a batch, up to kMaxPhases of them to a launch.
struct VotePlan {
  std::vector<VoteLaunch> parts;
  int resident = 0;  // workgroups of the kernel that the device holds at once
};
bool plan_vote_launches(const ts_config* cfg, const ts_batch* bt, VotePlan* plan);

// The per-workgroup statistics are their own flags (a sum of exponentials is never
// zero): the chunks a launch may fill have to be zero before it, `chunks` of every
// (request, head) row.
static ZeroRegion partials_zero_region(const SelectWorkspace& w, void* workspace, int batch, int heads,
                                       int chunks) {
  ZeroRegion z;
  z.base = (uint32_t*)((char*)workspace + w.partials);
  z.stride = (int64_t)kSelMaxChunks * 2;
  z.words = std::min(chunks, kSelMaxChunks) * 2;
  z.count = batch * heads;
  return z;
}
static ZeroRegion stats_zero_region(const SelectWorkspace& w, void* workspace, int batch, int heads) {
  ZeroRegion z;  // the live words of the 64 replicas
  z.base = (uint32_t*)((char*)workspace + w.stats);
  z.stride = w.stats_stride;
  z.words = batch * heads * 2;
  z.count = kSyncSlots;
  return z;
}
static ZeroRegion sync_zero_region(const SelectWorkspace& w, void* workspace, int areas) {
  ZeroRegion z;
  z.base = (uint32_t*)((char*)workspace + w.sync);
  z.stride = kSyncSlotWords;
  z.words = kSyncLiveWords;
  z.count = (kSyncSlots + 1) * areas;
  return z;
}

void select_zero_regions(const ts_config* cfg, const SelectWorkspace& w, void* workspace, int batch,
                         ZeroSet* zero) {
  ZeroRegion counters;
  counters.base = (uint32_t*)((char*)workspace + w.counters);
  counters.words = batch * kSelCounterWords;
  counters.stride = counters.words;
  counters.count = 1;
  zero->add(counters);
  zero->add(stats_zero_region(w, workspace, batch, cfg->num_heads));
  zero->add(sync_zero_region(w, workspace, 1));
  zero->add(partials_zero_region(w, workspace, batch, cfg->num_heads, w.clear_chunks));
}

void score_votes_zero_regions(const ts_config* cfg, const ts_batch* bt, const SelectWorkspace& w,
                              void* workspace, ZeroSet* zero) {
  VotePlan plan;
  int chunks = 0;
  if (plan_vote_launches(cfg, bt, &plan))
    for (const VoteLaunch& v : plan.parts) chunks = std::max(chunks, v.table_chunks);
  zero->add(stats_zero_region(w, workspace, bt->batch, cfg->num_heads));
  zero->add(sync_zero_region(w, workspace, bt->batch));
  zero->add(partials_zero_region(w, workspace, bt->batch, cfg->num_heads, chunks));
}

bool vote_launches_planned(const ts_config* cfg, const ts_batch* bt) {
  if (bt->max_seq_len - cfg->n_init - cfg->n_local <= 0) return false;
  VotePlan plan;
  return plan_vote_launches(cfg, bt, &plan);
}
bool vote_launches_planned(const ts_config* cfg, int batch, int max_seq_len) {
  ts_batch bt{};
  bt.batch = batch;
  bt.max_seq_len = max_seq_len;
  return vote_launches_planned(cfg, &bt);
}

const uint32_t* score_votes_fault_word(const ts_config* cfg, int batch, int max_seq_len,
                                       const void* workspace) {
  return (const uint32_t*)((const char*)workspace + select_workspace(cfg, batch, max_seq_len, true).sync);
}

__global__ __launch_bounds__(256) void select_zero_kernel(ZeroSet zero) {
  clear_regions(zero, (int64_t)blockIdx.x * 256 + threadIdx.x, (int64_t)gridDim.x * 256);
}
int launch_select_zero(const ZeroSet& zero, hipStream_t stream) {
  TS_REQUIRE(!zero.overflow, TS_EINVAL, "internal: more than %d regions to clear in one launch", kZeroRegions);
  const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>(1024, ceil_div(zero.total(), 1024)));
  hipLaunchKernelGGL(select_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, zero);
  return check_launch("select_zero_kernel");
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

int launch_select(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                  int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
                  int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
                  int64_t vote_stride, void* workspace, uint32_t* clear, int clear_per_req,
                  hipStream_t stream, uint64_t wait_ticks, uint32_t absent,
                  const UnrotatedQuery* unrotated) {
  // (requests may be skipped when the caller brings hit flags: the selection cache)
  const SelectWorkspace w = select_workspace(cfg, bt->batch, bt->max_seq_len, false, hit != nullptr);
  TS_REQUIRE(w.tokens_per_block > 0, TS_ESHAPE, "fused selection: unsupported shape");
  char* ws = (char*)workspace;
  ScoreArgs a = selection_args(cfg, bt, qf, k_pool, pool_rows, hit, (float*)(ws + w.partials),
                               w.tokens_per_block);
  a.nchunks = kSelMaxChunks;  // the row of a (request, head) pair in the statistics' table
  if (unrotated) {
    a.q_raw = (const uint16_t*)unrotated->q;
    a.q_cos = unrotated->cos;
    a.q_sin = unrotated->sin;
  }
  a.sync = (uint32_t*)(ws + w.sync);
  a.stats = (float*)(ws + w.stats);
  a.stats_stride = w.stats_stride;
  a.votes = votes;
  a.vote_stride = vote_stride;
  a.counters = (uint32_t*)(ws + w.counters);
  a.block_counts = (uint2*)(ws + w.block_counts);
  a.short_list = (uint2*)(ws + w.short_list);
  a.hint = bt->threshold_hint;
  a.band_above = (uint32_t*)(ws + w.band_above);
  a.band_slots = (uint4*)(ws + w.band_slots);
  a.sel = sel;
  a.sel_pos = sel_pos;
  a.sel_stride = sel_stride;
  a.sel_len = sel_len;
  a.topk_cache = cache ? cache->topk_cache : nullptr;
  a.cache_len = cache ? cache->cache_len : nullptr;
  a.clear = clear;
  a.clear_per_req = clear_per_req;
  a.spin_ticks = wait_ticks;
  a.absent = absent;
  a.fault_out = bt->fault;
  a.pool_kernel = cfg->pool_kernel;
  a.pool_votes = (float*)(ws + w.pool_votes);
  a.pool_stride = w.pool_stride;
  const void* fn = fused_kernel_of(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads);
  // One-dimensional: the kernel deals these workgroups over the requests that select.
  a.batch = bt->batch;
  const dim3 grid((unsigned)(w.blocks_per_req * bt->batch), 1u);
  void* params[] = {(void*)&a};
  // An ordinary launch: the grid was sized to be resident all at once, which holds
  // as long as the device runs nothing else beside this stream.  (The cooperative
  // launch API would guarantee it, at some 25 us of extra launch latency.)
  const hipError_t e =
      hipLaunchKernel(fn, grid, dim3(256), params, w.lds_bytes, stream);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(TS_EHIP, "fused selection launch: %s", hipGetErrorString(e));
  }
  return TS_OK;
}

// The votes-only form: consecutive requests are packed into phases by what they can
// hold -- the host's upper bounds of the lengths (ts_batch.host_seq_lens) where it has
// them, max_seq_len else -- as many as fit half the device (all of it, when a request
// needs more) with the most tokens per workgroup that the LDS takes.  One launch holds
// the workgroups of many phases, one after the other in a one-dimensional grid.  The
// device starts the workgroups of a grid in the order of their numbers as room becomes
// free (of those that go to one XCD, every eighth): with phases of half the device two
// of them are resident side by side, and when the workgroups of the earlier one leave,
// those of the next but one take their places.  A phase ends with the memory idle (the
// statistics on their way, scores turned into votes); the other phase streams
// meanwhile.  Two phases that start together would also wait together, so the second
// phase is given about half the candidates of a full one.  A workgroup without
// candidates (the bound was above the length) leaves at once and is not on the phase's
// team.  Nothing can wait forever: the workgroups of the earliest unfinished phase wait
// for each other only, and all of them have been started, since every workgroup started
// before them has left and fewer than fit are left to start.
// (A grid [chunks of the longest, requests] of a group of requests that must all be
// resident at once is not an alternative: its members have gaps between them and do not
// spread evenly over the XCDs; such launches were seen to wait for room that never came.)
bool plan_vote_launches(const ts_config* cfg, const ts_batch* bt, VotePlan* plan) {
  plan->parts.clear();
  if (!fused_kernels_enabled()) return false;
  if (cfg->num_heads > kMaxHeads || cfg->pool_kernel > 256) return false;
  const int fixed = cfg->n_init + cfg->n_local;
  auto bound = [&](int b) { return bt->host_seq_lens ? std::min(bt->host_seq_lens[b], bt->max_seq_len) : bt->max_seq_len; };
  auto candidates = [&](int b) { return std::max(bound(b) - fixed, 0); };
  int longest_n = 0;
  for (int b = 0; b < bt->batch; ++b) longest_n = std::max(longest_n, candidates(b));
  // The most tokens a workgroup of either size takes, and what is resident of them.
  auto size_up = [&](bool large, int* capacity_out) {
    *capacity_out = fused_capacity(cfg, /*packed=*/true, large);
    int most = 64;
    while (fused_lds_bytes(most + 64, cfg->num_heads) <= fused_stage_bytes(large) &&
           most + 64 <= pooling_tokens_cap(cfg))
      most += 64;
    return (*capacity_out > 0 && fused_lds_bytes(most, cfg->num_heads) <= fused_stage_bytes(large)) ? most : 0;
  };
  int capacity = 0;
  int tpb_max = size_up(false, &capacity);
  // The large workgroups when the longest request takes more than half of the device.
  if (tpb_max == 0 || ceil_div(longest_n, tpb_max) > capacity / 2) {
    int capacity_large = 0;
    const int most = size_up(true, &capacity_large);
    if (most > tpb_max) {
      tpb_max = most;
      capacity = capacity_large;
    }
  }
  if (tpb_max == 0) return false;
  plan->resident = capacity;
  // Phases of half the device when every request fits that.
  bool halves = bt->batch >= 2;
  for (int b = 0; b < bt->batch && halves; ++b)
    if (ceil_div(candidates(b), tpb_max) > capacity / 2) halves = false;
  const int room_full = halves ? capacity / 2 : capacity;
  for (int first = 0; first < bt->batch;) {
    // (the second phase: half a phase, see above)
    const bool shorter = halves && plan->parts.size() == 1;
    int64_t wgs = 0;
    int last = first, longest = 0;
    for (int pass = shorter ? 0 : 1; pass < 2 && last == first; ++pass) {
      const int64_t room = pass == 0 ? room_full / 2 : room_full;
      for (; last < bt->batch && last - first < kMaxPacked; ++last) {
        const int64_t more = ceil_div(candidates(last), tpb_max);
        if (wgs + more > room) break;
        wgs += more;
        longest = std::max(longest, bound(last));
      }
    }
    if (last == first) return false;  // a single request does not fit the device
    // Every workgroup takes as many tokens as the LDS holds (the statistics' table of a
    // request has room for kSelMaxChunks chunks): the fewer workgroups a phase has, the
    // sooner those of the next one find room, and the less each token carries of what a
    // workgroup does once (queries, statistics, the wait for them).
    const int tpb = tpb_max;
    if (ceil_div(longest, tpb) > kSelMaxChunks) return false;
    if (wgs > 0)  // (nothing to do for requests that are all sink and local window)
      plan->parts.push_back(VoteLaunch{first, last - first, tpb, (int)wgs, (int)ceil_div(longest, tpb)});
    first = last;
  }
  return true;
}

int launch_score_votes(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                       int64_t pool_rows, const int32_t* skip, float* votes, int64_t vote_stride,
                       uint32_t* hist_ws, size_t hist_ws_stride, void* workspace, hipStream_t stream) {
  VotePlan plan;
  TS_REQUIRE(plan_vote_launches(cfg, bt, &plan), TS_ESHAPE,
             "fused scoring + vote: not even one request of %d tokens fits", bt->max_seq_len);
  // Offsets of the pieces: those of the whole batch's workspace, whatever the launches.
  const SelectWorkspace all = select_workspace(cfg, bt->batch, bt->max_seq_len, true);
  char* ws = (char*)workspace;
  const void* fn = fused_kernel_of(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads, true);
  const int per_launch = kMaxPhases;
  for (size_t at = 0; at < plan.parts.size(); at += per_launch) {
    const VoteLaunch& v = plan.parts[at];
    ScoreArgs a = selection_args(cfg, bt, qf, k_pool, pool_rows, skip, (float*)(ws + all.partials),
                                 v.tokens_per_block);
    a.nchunks = kSelMaxChunks;
    a.sync = (uint32_t*)(ws + all.sync) + at * kSyncWords;  // one rendezvous area per part
    a.fault_word = (uint32_t*)(ws + all.sync);
    a.stats = (float*)(ws + all.stats);
    a.stats_stride = all.stats_stride;
    a.votes = votes;
    a.vote_stride = vote_stride;
    a.counters = (uint32_t*)(ws + all.counters);
    a.spin_ticks = select_wait_ticks(bt);
    a.absent = (uint32_t)std::max(bt->absent_workgroups, 0);
    a.fault_out = bt->fault;
    a.pool_kernel = cfg->pool_kernel;
    a.pool_votes = (float*)(ws + all.pool_votes);
    a.pool_stride = all.pool_stride;
    a.batch_offset = v.first;
    a.hist_ws = hist_ws;
    a.hist_ws_stride = hist_ws_stride;
    a.resident = plan.resident;
    int tpb_lds = v.tokens_per_block;
    dim3 grid;
    {
      const int phases = (int)std::min<size_t>(per_launch, plan.parts.size() - at);
      const int fixed = cfg->n_init + cfg->n_local;
      a.nphases = phases;
      int workgroups = 0;
      for (int p = 0; p < phases; ++p) {
        const VoteLaunch& part = plan.parts[at + p];
        VotePhase& ph = a.phases[p];
        ph.tokens_per_block = part.tokens_per_block;
        ph.first = part.first;
        ph.requests = part.requests;
        ph.first_workgroup = workgroups;
        ph.pack_first[0] = 0;
        for (int r = 0; r < part.requests; ++r) {
          const int len = bt->host_seq_lens ? std::min(bt->host_seq_lens[part.first + r], bt->max_seq_len)
                                            : bt->max_seq_len;
          const int cand = std::max(len - fixed, 0);
          ph.pack_first[r + 1] = ph.pack_first[r] + (int)ceil_div(cand, part.tokens_per_block);
        }
        workgroups += part.workgroups;
        tpb_lds = std::max(tpb_lds, part.tokens_per_block);
      }
      grid = dim3((unsigned)workgroups, 1u);
    }
    void* params[] = {(void*)&a};
    const hipError_t e = hipLaunchKernel(fn, grid, dim3(256), params,
                                         fused_lds_bytes(tpb_lds, cfg->num_heads), stream);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(TS_EHIP, "fused scoring + vote launch: %s", hipGetErrorString(e));
    }
  }
  return TS_OK;
}

}  // namespace ts

using namespace ts;

extern "C" {

int ts_set_fused_select(int enable) { return set_fused_select(enable); }

size_t ts_score_partials_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  // A bound that never shrinks when max_seq_len grows, unlike the number of workgroups
  // itself (the candidates per workgroup move in steps of 64), so that a buffer sized
  // for the longest context serves every shorter one: 256 workgroups are aimed at (the
  // bound leaves room for twice that), more only once a workgroup holds as many candidates
  // as its LDS takes.
  const int64_t cap = std::max<int64_t>((16384 / cfg->num_heads) / 64 * 64, 64);
  const size_t nchunks = (size_t)std::max<int64_t>(520, ceil_div(max_seq_len, cap) + 8);
  return align_up((size_t)batch * cfg->num_heads * nchunks * 2 * sizeof(float), 256);
}

int ts_score(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
             int64_t pool_rows, const int32_t* skip, float* scores, int64_t score_stride,
             float* partials, size_t partials_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(qf && k_pool && scores && partials, TS_EINVAL, "ts_score: NULL tensor argument");
  TS_REQUIRE_ALIGNED(qf, 16, "qf");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(scores, 16, "scores");
  TS_REQUIRE_ALIGNED(partials, 16, "partials");
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
  return vote_launches_planned(cfg, batch, max_seq_len) ? 1 : 0;
}

int ts_score_vote(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                  int64_t pool_rows, const int32_t* skip, float* votes, int64_t vote_stride,
                  void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(qf && k_pool && votes && workspace, TS_EINVAL, "ts_score_vote: NULL argument");
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(qf, 16, "qf");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  TS_REQUIRE(ts_score_vote_supported(cfg, bt->batch, bt->max_seq_len), TS_ESHAPE,
             "ts_score_vote: not even one request of %d tokens fits the LDS of the device (or "
             "pool_kernel is above 256, or the fused kernels are switched off); use ts_score + ts_vote",
             bt->max_seq_len);
  const SelectWorkspace w = select_workspace(cfg, bt->batch, bt->max_seq_len, true);
  TS_REQUIRE(workspace_bytes >= w.total, TS_EWORKSPACE, "ts_score_vote: workspace %zu bytes < required %zu",
             workspace_bytes, w.total);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  if (max_n <= 0) return TS_OK;
  ZeroSet zero;
  score_votes_zero_regions(cfg, bt, w, workspace, &zero);
  TS_TRY(launch_select_zero(zero, (hipStream_t)stream));
  return launch_score_votes(cfg, bt, qf, k_pool, pool_rows, skip, votes, vote_stride, nullptr, 0,
                            workspace, (hipStream_t)stream);
}

int ts_select_supported(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  return fused_tokens_per_block(cfg, batch, max_seq_len, false, nullptr, false, nullptr) > 0 ? 1 : 0;
}

size_t ts_select_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  return select_workspace(cfg, batch, max_seq_len).total;
}

// Argument checks shared by the three forms of the call.
static int check_select(const ts_config* cfg, const ts_batch* bt, const void* workspace,
                        size_t workspace_bytes, SelectWorkspace* w_out) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  TS_REQUIRE(workspace != nullptr, TS_EINVAL, "ts_select: NULL workspace");
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  const SelectWorkspace w = select_workspace(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(w.tokens_per_block > 0, TS_ESHAPE,
             "ts_select: batch %d x %d tokens does not fit one co-resident grid (or pool_kernel is "
             "above 256); use ts_score + ts_vote + ts_topk_ragged",
             bt->batch, bt->max_seq_len);
  TS_REQUIRE(workspace_bytes >= w.total, TS_EWORKSPACE, "ts_select: workspace %zu bytes < required %zu",
             workspace_bytes, w.total);
  *w_out = w;
  return TS_OK;
}

int ts_select_clear(const ts_config* cfg, const ts_batch* bt, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream) {
  SelectWorkspace w;
  TS_TRY(check_select(cfg, bt, workspace, workspace_bytes, &w));
  ZeroSet zero;
  select_zero_regions(cfg, w, workspace, bt->batch, &zero);
  return launch_select_zero(zero, (hipStream_t)stream);
}

int ts_select_cleared_bounded(const ts_config* cfg, const ts_batch* bt, const void* qf,
                              const void* k_pool, int64_t pool_rows, const int32_t* hit,
                              const ts_selcache* cache, int32_t* sel, int32_t* sel_pos,
                              int64_t sel_stride, int32_t* sel_len, float* votes,
                              int64_t vote_stride, void* workspace, size_t workspace_bytes,
                              uint64_t wait_ticks, int32_t absent_workgroups, ts_stream_t stream) {
  SelectWorkspace w;
  TS_REQUIRE(wait_ticks >= 1 && absent_workgroups >= 0, TS_EINVAL,
             "ts_select: wait_ticks %llu / absent_workgroups %d out of range",
             (unsigned long long)wait_ticks, absent_workgroups);
  TS_TRY(check_select(cfg, bt, workspace, workspace_bytes, &w));
  TS_REQUIRE(qf && k_pool && sel && sel_pos && sel_len, TS_EINVAL, "ts_select: NULL tensor argument");
  TS_REQUIRE_ALIGNED(qf, 16, "qf");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const int max_sel = cfg->n_init + cfg->top_k + cfg->n_local;
  TS_REQUIRE(sel_stride >= max_sel, TS_EWORKSPACE, "sel_stride %lld < n_init+top_k+n_local = %d",
             (long long)sel_stride, max_sel);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(votes == nullptr || vote_stride >= max_n, TS_EWORKSPACE,
             "vote_stride %lld < max candidates %d", (long long)vote_stride, max_n);
  TS_REQUIRE(hit == nullptr || cache != nullptr, TS_EINVAL,
             "ts_select: hit flags need the selection cache");
  if (cache)
    TS_REQUIRE(cache->topk_cache && cache->cache_len, TS_EINVAL,
               "ts_select: selection cache has a NULL array");
  return launch_select(cfg, bt, qf, k_pool, pool_rows, hit, cache, sel, sel_pos, sel_stride, sel_len,
                       votes, vote_stride, workspace, nullptr, 0, (hipStream_t)stream, wait_ticks,
                       (uint32_t)absent_workgroups);
}

int ts_select_cleared(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                      int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
                      int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
                      int64_t vote_stride, void* workspace, size_t workspace_bytes,
                      ts_stream_t stream) {
  return ts_select_cleared_bounded(cfg, bt, qf, k_pool, pool_rows, hit, cache, sel, sel_pos, sel_stride,
                                   sel_len, votes, vote_stride, workspace, workspace_bytes,
                                   bt ? select_wait_ticks(bt) : 1, bt ? std::max(bt->absent_workgroups, 0) : 0,
                                   stream);
}

int ts_select(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
              int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
              int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
              int64_t vote_stride, void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(ts_select_clear(cfg, bt, workspace, workspace_bytes, stream));
  return ts_select_cleared(cfg, bt, qf, k_pool, pool_rows, hit, cache, sel, sel_pos, sel_stride,
                           sel_len, votes, vote_stride, workspace, workspace_bytes, stream);
}

int ts_paged_matmul(const void* query, const void* token, int64_t pool_rows,
                    const int32_t* indices, void* scores, int32_t scores_dtype, int64_t n,
                    int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                    ts_stream_t stream) {
  TS_REQUIRE(query && token && indices && scores, TS_EINVAL, "ts_paged_matmul: NULL tensor argument");
  TS_REQUIRE_ALIGNED(query, 16, "query");
  TS_REQUIRE_ALIGNED(token, 16, "token");
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
