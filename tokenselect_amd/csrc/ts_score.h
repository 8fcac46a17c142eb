// Arguments of the scoring kernels and the workspace of the fused selection, shared
// between the scoring entry points and the per-layer driver.
#pragma once

#include "ts_grid.h"
#include "ts_topk.h"

namespace ts {

constexpr int kMaxPacked = 8;   // requests per phase of a launch of the votes-only form
constexpr int kMaxPhases = 24;  // phases per launch

// One phase of a votes-only launch: `requests` requests from `first` on share the workgroups
// [first_workgroup, next phase's first_workgroup) of the grid, request r owning those from
// pack_first[r] on (relative to the phase).
struct VotePhase {
  int tokens_per_block, first, requests, first_workgroup;
  int pack_first[kMaxPacked + 1];
};

struct ScoreArgs {
  const uint16_t* qf;      // [B,H,128] bf16 rotated fingerprints
  // Single-launch selection only: when q_raw is set, qf is not read; the kernel rotates
  // q_raw [B,H,128] (un-rotated bf16) itself with the [128] rows q_cos / q_sin, bit-identical
  // to what the rotation kernel would have written to qf.
  const uint16_t* q_raw;
  const float* q_cos;
  const float* q_sin;
  const uint16_t* k_pool;  // [pool_rows,Hkv,128] bf16
  uint32_t pool_rows;
  const int32_t* seq_lens;
  const int32_t* table;
  int64_t table_stride;
  const int32_t* k_per_req;
  const int32_t* skip;  // per request: 1 = selection-cache hit, nothing to score
  int n_init, n_local, top_k, page_size, page_shift, max_seq_len;
  int64_t direct_n;  // >= 0: paged_matmul mode, candidates are table[0..direct_n)
  void* scores;
  int64_t score_stride;  // elements between head rows
  float* partials;       // [B,H,nchunks,2] or NULL
  int nchunks;
  int tokens_per_block;
  int num_heads;
  int head_map;
  // Fused selection only.
  uint32_t* sync;         // rendezvous area (ts_grid.h), live words zero at launch
  float* stats;           // [kSyncSlots replicas][stats_stride]: [B,H,2] merged (max, sum exp), by
                          // head, zero at launch
  int64_t stats_stride;   // floats between replicas
  float* votes;           // [B,vote_stride] copy of the votes, or NULL
  int64_t vote_stride;
  uint32_t* counters;     // [B][kSelCounterWords] zero at launch
  uint2* block_counts;    // [B][gridDim.x] (selected for sure, ties at the k-th key)
  uint2* short_list;      // [B][kSelListParts][kSelListCap] (key, position) of the threshold bin
  int32_t* sel;           // outputs of the selection, as for ts_topk_ragged
  int32_t* sel_pos;
  int64_t sel_stride;
  int32_t* sel_len;
  int32_t* topk_cache;    // selection cache to refresh on a miss, or NULL
  int32_t* cache_len;
  uint32_t* clear;        // words to clear for the next kernel of the stream, or NULL
  int clear_per_req;
  uint64_t spin_ticks;    // bound of a grid-wide wait, in 100 MHz ticks
  int batch_offset;       // request index of the launch's first request
  int batch;              // requests of the launch (the single-launch selection deals its
                          // one-dimensional grid over those of them that select)
  // Votes-only form of the fused kernel (a kernel instantiation of its own): the launch
  // ends with the votes in memory and their first-level histogram added to the top-k
  // workspace.  A one-dimensional grid holds the workgroups of `nphases` phases one after
  // the other, each phase a group of requests that fits half the device (or all of it).
  // A workgroup serves one phase; one without candidates (the length was below the bound
  // the phase was sized by) leaves at once and is not on the phase's team.  Phase p's
  // rendezvous area is sync + p * kSyncWords.
  int nphases;
  int resident;           // workgroups of the launch that the device holds at once
  VotePhase phases[kMaxPhases];
  uint32_t* hist_ws;      // per-request top-k workspace (ts_topk.h) whose hist0 is counted into, or NULL
  size_t hist_ws_stride;
  uint32_t* fault_word;   // votes-only: the word the kernels after this one consult
  uint32_t absent;        // team members that never arrive (tests of the give-up path)
  uint32_t* fault_out;    // caller's word, set to 1 when a wait gave up, or NULL
  int32_t* hint;          // [B] threshold bin + 1 of the last selection (0: none), or NULL
  uint32_t* band_above;   // [B][kBandBins][kSelMaxChunks]: tokens of a workgroup above a band bin << 16 | in it
  uint4* band_slots;      // [B][kBandBins][kSelMaxChunks]: kBandSlots packed candidates
  int pool_kernel;        // max-pool window over the votes (tr.py:366-369), <= 0: off
  float* pool_votes;      // [B,pool_stride] un-pooled votes exchanged between workgroups
  int64_t pool_stride;
};

// Selection counters of one request, in 32-bit words.  The first histogram is kept
// in kSelHistCopies copies (workgroup x adds to copy x % copies): the votes of a
// request fall into a few dozen adjacent bins, i.e. one or two cache lines, and
// hundreds of workgroups adding to the same line serialise in memory.
constexpr int kSelHistCopies = 16;
constexpr int kSelHist0 = 0;                           // copies x 2048, top 11 key bits
// Second level (next 11 bits inside bin t0), needed when the votes are nearly uniform
// and t0 holds tens of thousands of candidates: that many adds to the 64 lines of a
// single copy take 20 us, hence copies here as well.
constexpr int kSelHist1Copies = 8;
constexpr int kSelHist1 = kSelHistCopies * kTopkBins;             // copies x 2048
constexpr int kSelHist2 = kSelHist1 + kSelHist1Copies * kTopkBins;  // 1024, last 10 bits inside (t0, t1)
// Highest occupied bin of hist0, one word per copy, 128 bytes apart (hundreds of
// read-modify-writes of one address, or one line, take microseconds).
constexpr int kSelMaxBin = kSelHist2 + 1024;
// Once at most kSelListCap candidates are left in the threshold bin they are listed
// instead of being resolved by further histogram levels; the list is kept in parts
// with a fill counter each (128 bytes apart), workgroup x appending to part x % parts.
constexpr int kSelListCap = 256;
constexpr int kSelListParts = 8;
constexpr int kSelListCount = kSelMaxBin + kSelHistCopies * 32;
// With a hint of where the threshold bin is going to be (ts_batch.threshold_hint: the bin of
// the request's previous selection on the same layer), every workgroup publishes, together
// with its histogram and before the first rendezvous, what the last round would otherwise
// need a rendezvous of its own for, for each of the kBandBins bins around the hint: one word
// with the number of its tokens above that bin and of its candidates in it; those
// candidates (up to kBandSlots, packed into 32 bits each: the low 21 key bits and the
// token's index in the workgroup, which is why the band needs workgroups of at most 1024
// tokens; into a 16-byte piece of its own, no counter to reserve from, and only the entries
// the word counts are ever read, so nothing is cleared); and its counts of the band's bins
// added to a small histogram of the band (kBandHistCopies copies a line apart, slot
// kBandBins of each: the tokens above the band).  After the rendezvous the small histogram
// says whether the threshold bin lies in the band, and if no workgroup had more candidates
// in it than slots, the selection is through: one rendezvous, and a fraction of the
// histogram to read.  Every memory-side atomic counts here (a few thousand of them in a
// microsecond are what the device serves): a narrow band, and nothing written that is empty.
constexpr int kBandBins = 8;
constexpr int kBandBelow = 4;   // the band is [hint - kBandBelow, hint - kBandBelow + kBandBins)
constexpr int kBandSlots = 4;   // candidates a workgroup can publish per bin (one 16-byte piece)
constexpr int kBandMaxTokens = 1024;  // tokens per workgroup the packed index can address
constexpr int kBandHistCopies = 32;   // one 128-byte line each: adds to one line are served one by one
constexpr int kSelBandHist = kSelListCount + kSelListParts * 32;  // copies x 32 words (kBandBins + 1 live)
constexpr int kSelCounterWords = kSelBandHist + kBandHistCopies * 32;

// Workgroups of one request the workspace of ts_select is laid out for (the device keeps
// at most 512 resident at once).
constexpr int kSelMaxChunks = 1024;

// Workspace of ts_select, carved in this order (256-byte aligned pieces).
struct SelectWorkspace {
  size_t partials, counters, stats, block_counts, short_list, band_above, band_slots, pool_votes, sync,
      total;  // sync stays last
  int64_t stats_stride;
  int64_t pool_stride;
  int tokens_per_block;  // 0: the shape does not fit the fused kernel
  int blocks_per_req;
  int clear_chunks;      // per-workgroup statistics of a (request, head) row to clear before a launch
  size_t lds_bytes;      // dynamic LDS of the launch (decides how many workgroups share a CU)
};
// ignore_switch: lay out as if ts_set_fused_select were on (for sizing a workspace that
// must serve both settings).
// may_skip: requests of the launch may be skipped on the device (selection cache), which
// decides between one and two workgroups per CU; the layout does not depend on it.
SelectWorkspace select_workspace(const ts_config* cfg, int batch, int max_seq_len,
                                 bool ignore_switch = false, bool may_skip = false);

// Regions the kernel before ts_select on the stream has to clear (counters, replicas
// of the merged statistics, rendezvous words, the per-workgroup statistics), in the form
// the rotation kernel takes them.
void select_zero_regions(const ts_config* cfg, const SelectWorkspace& w, void* workspace, int batch,
                         ZeroSet* zero);

// Clears the regions (the stand-alone form of what the rotation kernel does on the side).
int launch_select_zero(const ZeroSet& zero, hipStream_t stream);

// Bound of a grid-wide wait of the fused kernels in ticks of the 100 MHz clock: the
// caller's ts_batch.wait_us, by default TS_DEFAULT_WAIT_US (10 ms).
static inline uint64_t select_wait_ticks(const ts_batch* bt) {
  return (uint64_t)(bt->wait_us ? bt->wait_us : TS_DEFAULT_WAIT_US) * 100ull;
}

// Whether the fused kernels (ts_select, the votes-only form) may serve on this thread
// right now: the process-wide switch, unless a call is running that asked for the
// separate kernels (ts_batch.separate_kernels).  SeparateKernelsScope is that call's guard.
bool fused_kernels_enabled();
struct SeparateKernelsScope {
  explicit SeparateKernelsScope(bool on);
  ~SeparateKernelsScope();
  bool was;
};

// Scores and votes of a batch of any size without the [H, n] scores in memory: the
// requests are served in phases whose scores fit the LDS of half the device (of all of it
// for a request that needs more), the workgroups of all phases in one launch of the fused
// kernel's votes-only form (score, statistics, votes, [max-pool]); the launch also counts
// the first histogram level of the top-k into hist_ws.  vote_launches_planned() tells
// whether the launcher's own plan serves the batch (every request fits the device, the
// fused kernels are switched on, the max-pool window fits): else the separate kernels
// serve.  The driver, the zero regions and the launch all go by that one plan.  The workspace is that of ts_select for the whole
// batch; the statistics (per workgroup and merged) and the rendezvous areas
// (score_votes_zero_regions) are zero.
bool vote_launches_planned(const ts_config* cfg, const ts_batch* bt);
bool vote_launches_planned(const ts_config* cfg, int batch, int max_seq_len);
void score_votes_zero_regions(const ts_config* cfg, const ts_batch* bt, const SelectWorkspace& w,
                              void* workspace, ZeroSet* zero);
int launch_score_votes(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                       int64_t pool_rows, const int32_t* skip, float* votes, int64_t vote_stride,
                       uint32_t* hist_ws, size_t hist_ws_stride, void* workspace, hipStream_t stream);
// The word the votes-only launches leave non-zero when a wait of theirs gave up.
const uint32_t* score_votes_fault_word(const ts_config* cfg, int batch, int max_seq_len,
                                       const void* workspace);

// Launch without the clearing pass: the regions above are known to be zero.
// A query that the selection kernel rotates itself (see ScoreArgs::q_raw).
struct UnrotatedQuery {
  const void* q;
  const float* cos;
  const float* sin;
};
int launch_select(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                  int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
                  int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
                  int64_t vote_stride, void* workspace, uint32_t* clear, int clear_per_req,
                  hipStream_t stream, uint64_t wait_ticks, uint32_t absent,
                  const UnrotatedQuery* unrotated = nullptr);

}  // namespace ts
