// Arguments of the scoring kernels, shared between the scoring entry points and
// the per-layer driver (which launches the fused score + vote form).
#pragma once

#include "ts_common.h"

namespace ts {

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
  // Fused score + vote only.
  uint32_t* sync;  // [0] arrival counter (zero at launch), [1] set when a wait gave up
  float* stats;  // [B,H,2] merged (max, sum exp), by head
  float* votes;
  int64_t vote_stride;
  uint32_t* topk_ws;  // per-request selection counters, zero at launch
  size_t topk_ws_stride;
  uint64_t spin_ticks;  // bound of the grid-wide wait, in 100 MHz ticks
};

// Tokens per workgroup of the fused form for this shape, or 0 when the batch does
// not fit one co-resident grid (the caller then runs the separate kernels).
int fused_tokens_per_block(const ts_config* cfg, int batch, int max_seq_len);

}  // namespace ts
