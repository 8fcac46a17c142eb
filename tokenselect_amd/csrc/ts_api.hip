// Host-side plumbing of the C ABI: error state, argument validation and the
// per-layer driver that chains the kernels of one decode step.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include "ts_score.h"
#include "ts_topk.h"

namespace ts {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TS_EHIP, "%s: %s", what, hipGetErrorString(e));
  return TS_OK;
}

bool group_supported(int num_kv_heads, int group) {
  bool kv_ok = num_kv_heads == 1 || num_kv_heads == 2 || num_kv_heads == 4 || num_kv_heads == 8;
  bool g_ok = group >= 1 && group <= 8;
  return kv_ok && g_ok;
}

int validate_config(const ts_config* cfg) {
  TS_REQUIRE(cfg != nullptr, TS_EINVAL, "config is NULL");
  TS_REQUIRE(cfg->head_dim == kHeadDim, TS_ESHAPE, "head_dim %d not supported (only 128)",
             cfg->head_dim);
  TS_REQUIRE(cfg->num_heads > 0 && cfg->num_kv_heads > 0, TS_EINVAL,
             "num_heads=%d num_kv_heads=%d must be positive", cfg->num_heads, cfg->num_kv_heads);
  TS_REQUIRE(cfg->num_heads % cfg->num_kv_heads == 0, TS_ESHAPE,
             "num_heads %d not a multiple of num_kv_heads %d", cfg->num_heads, cfg->num_kv_heads);
  TS_REQUIRE(group_supported(cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads), TS_ESHAPE,
             "unsupported head shape: num_kv_heads=%d (1,2,4,8) group=%d (1 to 8)",
             cfg->num_kv_heads, cfg->num_heads / cfg->num_kv_heads);
  TS_REQUIRE(page_shift_of(cfg->page_size) >= 0, TS_EINVAL, "page_size %d is not a power of two",
             cfg->page_size);
  TS_REQUIRE(cfg->n_init >= 0 && cfg->n_local >= 0 && cfg->top_k >= 1, TS_EINVAL,
             "n_init=%d n_local=%d top_k=%d out of range", cfg->n_init, cfg->n_local, cfg->top_k);
  TS_REQUIRE(cfg->head_map == TS_HEADMAP_MOD || cfg->head_map == TS_HEADMAP_DIV, TS_EINVAL,
             "head_map %d unknown", cfg->head_map);
  TS_REQUIRE(cfg->rope_mode == TS_ROPE_NONE || cfg->rope_mode == TS_ROPE_LLAMA, TS_EINVAL,
             "rope_mode %d unknown", cfg->rope_mode);
  if (cfg->rope_mode == TS_ROPE_LLAMA)
    TS_REQUIRE(cfg->rope_theta > 0.f && cfg->rope_scale > 0.f, TS_EINVAL,
               "rope_theta=%g rope_scale=%g must be positive", cfg->rope_theta, cfg->rope_scale);
  return TS_OK;
}

int validate_batch(const ts_config* cfg, const ts_batch* bt) {
  (void)cfg;
  TS_REQUIRE(bt != nullptr, TS_EINVAL, "batch is NULL");
  TS_REQUIRE(bt->batch >= 1, TS_EINVAL, "batch %d < 1", bt->batch);
  TS_REQUIRE(bt->max_seq_len >= 1, TS_EINVAL, "max_seq_len %d < 1", bt->max_seq_len);
  TS_REQUIRE(bt->seq_lens != nullptr, TS_EINVAL, "seq_lens is NULL");
  TS_REQUIRE(bt->table != nullptr, TS_EINVAL, "table is NULL");
  TS_REQUIRE(bt->batch == 1 || bt->table_stride * (int64_t)cfg->page_size >= bt->max_seq_len,
             TS_EINVAL, "table_stride %lld too small for max_seq_len %d at page_size %d",
             (long long)bt->table_stride, bt->max_seq_len, cfg->page_size);
  if (bt->host_seq_lens)
    for (int b = 0; b < bt->batch; ++b)
      TS_REQUIRE(bt->host_seq_lens[b] >= 0 && bt->host_seq_lens[b] <= bt->max_seq_len, TS_EINVAL,
                 "host_seq_lens[%d] = %d outside [0, max_seq_len %d]", b, bt->host_seq_lens[b],
                 bt->max_seq_len);
  return TS_OK;
}

int score_tokens_per_block(int64_t total_candidates, int num_heads) {
  // Aim for one workgroup per CU (256 of them), in 64-row steps (every wave on whole
  // 16-row tiles): two per CU would be resident (register budget), but half as many
  // concurrent streams read faster (C2: 50.3 -> 48.2 us, C1: 20.3 -> 18.9 us).  A
  // workgroup stages its fp32 scores in LDS, tokens * heads * 4 bytes <= 64 KB.
  int64_t cap = (16384 / (num_heads > 0 ? num_heads : 1)) / 64 * 64;
  if (cap < 64) cap = 64;
  int64_t per = ceil_div(ceil_div(total_candidates, 256), 64) * 64;
  if (per < 64) per = 64;
  if (per > cap) per = cap;
  return (int)per;
}

}  // namespace ts

using namespace ts;

extern "C" {

int ts_version(void) { return TS_VERSION; }

const char* ts_last_error(void) { return ts::g_error; }

int ts_check_config(const ts_config* cfg) { return validate_config(cfg); }

int64_t ts_score_stride(int32_t max_seq_len) {
  return ceil_div(max_seq_len > 0 ? max_seq_len : 1, 64) * 64;
}

// Workspace of ts_decode_layer, carved in this order (256-byte aligned pieces).
struct LayerWorkspace {
  size_t qf, hit, scores, stats, votes, pooled, partials, topk_ws, select_ws, attn_ws, total;
  size_t partials_bytes;
  int64_t score_stride;
  int32_t max_sel;
};

static LayerWorkspace layer_workspace(const ts_config* cfg, int32_t batch, int32_t max_seq_len,
                                      bool ignore_switch = false) {
  LayerWorkspace w;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t at = off;
    off += align_up(bytes, 256);
    return at;
  };
  const size_t B = (size_t)batch, H = (size_t)cfg->num_heads;
  w.score_stride = ts_score_stride(max_seq_len);
  w.max_sel = cfg->n_init + cfg->top_k + cfg->n_local;
  w.qf = take(B * H * kHeadDim * 2);
  w.hit = take(B * 4);
  w.scores = take(B * H * (size_t)w.score_stride * 4);
  w.stats = take(B * H * 2 * 4);
  w.votes = take(B * (size_t)w.score_stride * 4);
  w.pooled = take(cfg->pool_kernel > 0 ? B * (size_t)w.score_stride * 4 : 0);
  w.partials_bytes = ts_score_partials_bytes(cfg, batch, max_seq_len);
  w.partials = take(w.partials_bytes);
  w.topk_ws = take(ts_topk_workspace_bytes(cfg, batch, max_seq_len));
  w.select_ws = take(select_workspace(cfg, batch, max_seq_len, ignore_switch).total);
  {  // decode attention partials, or the staging area of the prefill attention
    const size_t decode = ts_attn_workspace_bytes(cfg, batch, w.max_sel);
    const size_t prefill = ts_prefill_attn_workspace_bytes(cfg, w.max_sel);
    w.attn_ws = take(decode > prefill ? decode : prefill);
  }
  w.total = off;
  return w;
}

static int layer_selection_form(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
static int layer_selection_form(const ts_config* cfg, const ts_batch* bt);

int ts_decode_layer_selection(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return -1;
  return layer_selection_form(cfg, batch, max_seq_len);
}

int ts_decode_layer_selection_of(const ts_config* cfg, const ts_batch* bt) {
  if (validate_config(cfg) != TS_OK || validate_batch(cfg, bt) != TS_OK) return -1;
  return layer_selection_form(cfg, bt);
}

size_t ts_decode_layer_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  if (validate_config(cfg) != TS_OK || batch < 1 || max_seq_len < 1) return 0;
  // A workspace sized for `batch` serves every smaller batch and both settings of
  // ts_set_fused_select: the pieces do not all grow with the batch (attention splits,
  // candidates per workgroup of the fused selection), so the largest layout is taken.
  size_t most = 0;
  for (int32_t b = 1; b <= batch; ++b) {
    const size_t need = layer_workspace(cfg, b, max_seq_len, /*ignore_switch=*/true).total;
    if (need > most) most = need;
  }
  return most;
}

// How ts_decode_layer selects for a shape: 2 = the single ts_select kernel, 1 = scores and
// votes as by ts_score_vote (a batch too large for one co-resident launch: its requests as
// phases of one launch), then the top-k kernels, 0 = ts_score, ts_vote and the top-k
// kernels (fused kernels switched off, a max-pool window above 256, a request that does
// not fit the device).
// The second form is decided by the plan its launcher is going to follow, so that the
// driver, the regions cleared for it and the launch cannot disagree.
static int layer_selection_form(const ts_config* cfg, const ts_batch* bt) {
  SeparateKernelsScope separate(bt->separate_kernels != 0);
  if (select_workspace(cfg, bt->batch, bt->max_seq_len).tokens_per_block > 0) return 2;
  return vote_launches_planned(cfg, bt) ? 1 : 0;
}

static int layer_selection_form(const ts_config* cfg, int32_t batch, int32_t max_seq_len) {
  ts_batch bt{};
  bt.batch = batch;
  bt.max_seq_len = max_seq_len;
  return layer_selection_form(cfg, &bt);
}

// Decode (chunk_rows == 0: one query row per request, q_cos / q_sin are the [D] rows
// of position n_local) or one prefill chunk of a single request (chunk_rows > 0:
// q_cos / q_sin are the whole [table_rows, D] tables).
static int run_layer(const ts_config* cfg, const ts_batch* bt, const void* q, int32_t chunk_rows,
                     const float* q_cos, const float* q_sin, int64_t table_rows,
                     const void* k_pool, const void* v_pool, int64_t pool_rows,
                     const ts_selcache* cache, void* out, int32_t* sel, int32_t* sel_pos,
                     int64_t sel_stride, int32_t* sel_len, void* workspace, size_t workspace_bytes,
                     ts_stream_t stream, const StepStore* store = nullptr,
                     const ChunkStore* chunk_store = nullptr) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  SeparateKernelsScope separate(bt->separate_kernels != 0);
  TS_REQUIRE(q && q_cos && q_sin && k_pool && v_pool && out && sel && sel_pos && sel_len, TS_EINVAL,
             "layer: NULL tensor argument");
  TS_REQUIRE(store == nullptr || (cache != nullptr && chunk_rows == 0), TS_EINVAL,
             "internal: a store rides in the rotation + cache decision launch only");
  TS_REQUIRE(chunk_store == nullptr || chunk_rows > 0, TS_EINVAL,
             "internal: a chunk's store rides in the fingerprint launch only");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  LayerWorkspace w = layer_workspace(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE_ALIGNED(out, 16, "out");
  // The tie-break of the ragged top-k orders positions by two 10-bit digits.
  TS_REQUIRE(bt->max_seq_len - cfg->n_init - cfg->n_local <= (1 << 20), TS_ESHAPE,
             "layer: at most 2^20 candidates per request (max_seq_len %d)", bt->max_seq_len);
  TS_REQUIRE(sel_stride >= w.max_sel, TS_EWORKSPACE, "sel_stride %lld < n_init+top_k+n_local = %d",
             (long long)sel_stride, w.max_sel);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= w.total, TS_EWORKSPACE,
             "workspace %zu bytes < required %zu", workspace_bytes, w.total);
  if (cache)
    TS_REQUIRE(cache->q_cache && cache->topk_cache && cache->cache_len && cache->counters, TS_EINVAL,
               "selection cache has a NULL array");

  char* ws = (char*)workspace;
  void* qf = ws + w.qf;
  int32_t* hit = cache ? (int32_t*)(ws + w.hit) : nullptr;
  float* scores = (float*)(ws + w.scores);
  float* stats = (float*)(ws + w.stats);
  float* votes = (float*)(ws + w.votes);
  float* pooled = cfg->pool_kernel > 0 ? (float*)(ws + w.pooled) : nullptr;

  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  const SelectWorkspace fused = select_workspace(cfg, bt->batch, bt->max_seq_len);
  uint32_t* tickets = attn_tickets(cfg, bt->batch, w.max_sel, ws + w.attn_ws);

  // Fingerprint: every request's single decode row is rotated to n_local
  // (tr.py:381-388); the mean over one row is the row itself (tr.py:392).  The same
  // launch clears the counters the selection is going to add to.
  const bool one_launch = fused.tokens_per_block > 0;
  TopkArgs topk = make_topk_args(cfg, bt, pooled ? pooled : votes, w.score_stride, hit, cache, sel,
                                 sel_pos, sel_stride, sel_len, (uint32_t*)(ws + w.topk_ws));
  topk.clear = tickets;
  topk.clear_per_req = attn_tickets_per_request(cfg);
  // A batch too large for one launch of the selection: scores and votes still without
  // the [H, n] scores in memory, one launch per request, then the top-k kernels.
  const int vote_group = layer_selection_form(cfg, bt) == 1 ? 1 : 0;
  ZeroSet zero;
  if (one_launch) {
    select_zero_regions(cfg, fused, ws + w.select_ws, bt->batch, &zero);
  } else if (max_n > 0) {
    zero.add(topk_zero_region(topk, bt->batch));
    if (vote_group > 0) score_votes_zero_regions(cfg, bt, fused, ws + w.select_ws, &zero);
  }
  // A decode step without a selection cache whose single-launch selection finds its
  // counters zero (the caller says so: the attention kernel of its previous call, of the
  // same shape, cleared them on the side) starts with the selection kernel, which rotates
  // the query itself; this call's attention kernel clears the counters again.
  const bool plain_decode = one_launch && chunk_rows == 0 && !cache;
  const bool starts_with_selection = plain_decode && bt->workspace_clean != 0;
  if (starts_with_selection) {
  } else if (chunk_rows > 0) {
    // Chunk fingerprint: row i rotated to n_local + i, mean over the rows (tr.py:380-392).
    TS_TRY(launch_fingerprint(cfg, q, chunk_rows, q_cos, q_sin, table_rows, qf, zero,
                              (hipStream_t)stream, chunk_store));
  } else if (cache) {  // rotation and cache decision in one launch
    TS_TRY(launch_rope_selcache(cfg, bt, q, qf, q_cos, q_sin, cache, hit, bt->rerun ? sel_len : nullptr,
                                zero, (hipStream_t)stream, store));
  } else {
    TS_TRY(launch_rope(q, qf, q_cos, q_sin, nullptr, 1, bt->batch, cfg->num_heads, cfg->head_dim,
                       zero, (hipStream_t)stream));
  }
  if (cache && chunk_rows > 0)
    TS_TRY(launch_selcache(cfg, bt, qf, cache, hit, bt->rerun ? sel_len : nullptr, (hipStream_t)stream));
  const UnrotatedQuery unrotated{q, q_cos, q_sin};
  if (one_launch) {
    TS_TRY(launch_select(cfg, bt, qf, k_pool, pool_rows, hit, cache, sel, sel_pos, sel_stride, sel_len,
                         nullptr, 0, ws + w.select_ws, tickets, attn_tickets_per_request(cfg),
                         (hipStream_t)stream, select_wait_ticks(bt),
                         (uint32_t)(bt->absent_workgroups > 0 ? bt->absent_workgroups : 0),
                         starts_with_selection ? &unrotated : nullptr));
  } else if (vote_group > 0) {
    // With max-pooling the kernel writes the pooled votes (there is no un-pooled copy).
    TS_TRY(launch_score_votes(cfg, bt, qf, k_pool, pool_rows, hit, votes, w.score_stride, topk.ws,
                              topk.ws_stride, ws + w.select_ws, (hipStream_t)stream));
    topk.votes = votes;
    topk.fault = score_votes_fault_word(cfg, bt->batch, bt->max_seq_len, ws + w.select_ws);
    TS_TRY(launch_topk(topk, bt->batch, max_n, (hipStream_t)stream, true, true));
  } else {
    float* partials = (float*)(ws + w.partials);
    TS_TRY(ts_score(cfg, bt, qf, k_pool, pool_rows, hit, scores, w.score_stride, partials,
                    w.partials_bytes, stream));
    // The vote kernel counts the first histogram level of the selection as it goes
    // (not with max-pooling, which changes the votes afterwards).
    const bool zeroed = max_n > 0;
    TS_TRY(launch_vote(cfg, bt, scores, w.score_stride, partials, hit, stats, votes, pooled,
                       w.score_stride, zeroed ? topk.ws : nullptr, topk.ws_stride,
                       (hipStream_t)stream));
    TS_TRY(launch_topk(topk, bt->batch, max_n, (hipStream_t)stream, zeroed,
                       zeroed && cfg->pool_kernel <= 0));
  }
  if (chunk_rows > 0)
    return ts_sparse_prefill_attn(cfg, q, chunk_rows, k_pool, v_pool, pool_rows, sel, sel_len,
                                  w.max_sel, out, ws + w.attn_ws, w.total - w.attn_ws, stream);
  return launch_attn(cfg, q, k_pool, v_pool, pool_rows, sel, sel_stride, sel_len, bt->batch,
                     w.max_sel, out, ws + w.attn_ws, /*tickets_clear=*/true, (hipStream_t)stream,
                     plain_decode ? &zero : nullptr);
}

int ts_decode_layer(const ts_config* cfg, const ts_batch* bt, const void* q, const float* q_cos,
                    const float* q_sin, const void* k_pool, const void* v_pool,
                    int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                    int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream) {
  return run_layer(cfg, bt, q, 0, q_cos, q_sin, 1, k_pool, v_pool, pool_rows, cache, out, sel,
                   sel_pos, sel_stride, sel_len, workspace, workspace_bytes, stream);
}

// The reference's decode forward in one call (tr.py:777-825): store_kv_cache + add_k_cache,
// then selection and attention.  With a selection cache and slots chosen by the caller the
// store rides in the layer's first launch (the rotation and the cache decision, whose
// workgroup of a request stores that request's rows first); otherwise the two calls follow
// each other.
int ts_decode_step(const ts_config* cfg, const ts_batch* bt, const ts_new_kv* kv, const void* q,
                   const float* q_cos, const float* q_sin, void* k_pool, void* v_pool,
                   int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                   int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                   size_t workspace_bytes, ts_stream_t stream) {
  TS_REQUIRE(bt != nullptr && kv != nullptr, TS_EINVAL, "ts_decode_step: NULL batch / new K,V");
  TS_REQUIRE(bt->table != nullptr && bt->seq_lens != nullptr, TS_EINVAL, "ts_decode_step: NULL table / seq_lens");
  int32_t* table = const_cast<int32_t*>(bt->table);
  int32_t* seq_lens = const_cast<int32_t*>(bt->seq_lens);
  // (a call that repeats a step after a give-up does not append again: it is the layer alone)
  const bool rides = cache != nullptr && bt->rerun == 0;
  if (!rides) {
    if (bt->rerun == 0)
      TS_TRY(ts_kv_store(cfg, kv->k, kv->v, kv->out_cache_loc, kv->pages, k_pool, v_pool, pool_rows, table,
                         bt->table_stride, seq_lens, bt->batch, kv->max_tokens, stream));
    return run_layer(cfg, bt, q, 0, q_cos, q_sin, 1, k_pool, v_pool, pool_rows, cache, out, sel, sel_pos,
                     sel_stride, sel_len, workspace, workspace_bytes, stream);
  }
  // The checks ts_kv_store makes.
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(kv->k && kv->v && k_pool && v_pool, TS_EINVAL, "ts_decode_step: NULL tensor argument");
  TS_REQUIRE_ALIGNED(kv->k, 16, "k");
  TS_REQUIRE_ALIGNED(kv->v, 16, "v");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  if (kv->pages) {
    TS_REQUIRE(kv->pages->free_pages && kv->pages->free_count && kv->pages->ticket, TS_EINVAL,
               "ts_decode_step: page pool has a NULL array");
  } else {
    TS_REQUIRE(cfg->page_size == 1, TS_EINVAL, "ts_decode_step: pages of %d tokens need a page pool",
               cfg->page_size);
    TS_REQUIRE(kv->out_cache_loc != nullptr, TS_EINVAL, "ts_decode_step: NULL out_cache_loc and no page pool");
  }
  TS_REQUIRE(bt->batch >= 1 && pool_rows >= 1 && pool_rows <= 0x7fffffffLL && kv->max_tokens >= 1, TS_EINVAL,
             "ts_decode_step: batch=%d pool_rows=%lld max_tokens=%d out of range", bt->batch,
             (long long)pool_rows, kv->max_tokens);
  TS_REQUIRE(bt->batch == 1 || bt->table_stride * (int64_t)cfg->page_size >= kv->max_tokens, TS_EINVAL,
             "ts_decode_step: table_stride %lld x page_size %d < max_tokens %d", (long long)bt->table_stride,
             cfg->page_size, kv->max_tokens);
  StepStore st{};
  st.k = (const uint4*)kv->k;
  st.v = (const uint4*)kv->v;
  st.loc = kv->out_cache_loc;
  st.k_pool = (uint4*)k_pool;
  st.v_pool = (uint4*)v_pool;
  st.pool_rows = pool_rows;
  st.table = table;
  st.table_stride = bt->table_stride;
  st.seq_lens = seq_lens;
  st.row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  st.max_tokens = kv->max_tokens;
  if (kv->pages) {
    st.free_pages = kv->pages->free_pages;
    st.free_count = kv->pages->free_count;
    st.ticket = kv->pages->ticket;
    st.page_shift = page_shift_of(cfg->page_size);
  }
  return run_layer(cfg, bt, q, 0, q_cos, q_sin, 1, k_pool, v_pool, pool_rows, cache, out, sel, sel_pos,
                   sel_stride, sel_len, workspace, workspace_bytes, stream, &st);
}

// The layer split at the vote, for tensor parallelism (tr.py:361-364): every rank scores
// its own heads and holds partial votes; the ranks add them up (one all-reduce of the
// [B, vote_stride] votes, the caller's); every rank then selects the same tokens from
// the summed votes and attends with its own heads.
int ts_decode_layer_votes(const ts_config* cfg, const ts_batch* bt, const void* q, const float* q_cos,
                          const float* q_sin, const void* k_pool, int64_t pool_rows,
                          const ts_selcache* cache, float* votes, int64_t vote_stride,
                          void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  SeparateKernelsScope separate(bt->separate_kernels != 0);
  TS_REQUIRE(q && q_cos && q_sin && k_pool && votes, TS_EINVAL, "layer votes: NULL tensor argument");
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const LayerWorkspace w = layer_workspace(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= w.total, TS_EWORKSPACE,
             "workspace %zu bytes < required %zu", workspace_bytes, w.total);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  if (cache)
    TS_REQUIRE(cache->q_cache && cache->topk_cache && cache->cache_len && cache->counters, TS_EINVAL,
               "selection cache has a NULL array");
  ts_config plain = *cfg;  // the max-pool comes after the ranks' votes are added up
  plain.pool_kernel = -1;
  char* ws = (char*)workspace;
  void* qf = ws + w.qf;
  int32_t* hit = cache ? (int32_t*)(ws + w.hit) : nullptr;
  const SelectWorkspace fused = select_workspace(&plain, bt->batch, bt->max_seq_len);
  const int group = vote_launches_planned(&plain, bt) ? 1 : 0;
  ZeroSet zero;
  if (group > 0) score_votes_zero_regions(&plain, bt, fused, ws + w.select_ws, &zero);
  TS_TRY(launch_rope(q, qf, q_cos, q_sin, nullptr, 1, bt->batch, cfg->num_heads, cfg->head_dim,
                     zero, (hipStream_t)stream));
  if (cache) TS_TRY(ts_selcache_step(cfg, bt, qf, cache, hit, stream));
  if (max_n <= 0) return TS_OK;
  if (group > 0)
    return launch_score_votes(&plain, bt, qf, k_pool, pool_rows, hit, votes, vote_stride, nullptr, 0,
                              ws + w.select_ws, (hipStream_t)stream);
  float* partials = (float*)(ws + w.partials);
  TS_TRY(ts_score(&plain, bt, qf, k_pool, pool_rows, hit, (float*)(ws + w.scores), w.score_stride,
                  partials, w.partials_bytes, stream));
  return launch_vote(&plain, bt, (const float*)(ws + w.scores), w.score_stride, partials, hit,
                     (float*)(ws + w.stats), votes, nullptr, vote_stride, nullptr, 0, (hipStream_t)stream);
}

int ts_decode_layer_attend(const ts_config* cfg, const ts_batch* bt, const void* q, const float* votes,
                           int64_t vote_stride, const void* k_pool, const void* v_pool,
                           int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                           int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                           size_t workspace_bytes, ts_stream_t stream) {
  TS_TRY(validate_config(cfg));
  TS_TRY(validate_batch(cfg, bt));
  SeparateKernelsScope separate(bt->separate_kernels != 0);
  TS_REQUIRE(q && votes && k_pool && v_pool && out && sel && sel_pos && sel_len, TS_EINVAL,
             "layer attend: NULL tensor argument");
  TS_REQUIRE_ALIGNED(workspace, 256, "workspace");
  TS_REQUIRE_ALIGNED(q, 16, "q");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE_ALIGNED(out, 16, "out");
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL, TS_EINVAL, "pool_rows %lld out of range",
             (long long)pool_rows);
  const LayerWorkspace w = layer_workspace(cfg, bt->batch, bt->max_seq_len);
  TS_REQUIRE(workspace != nullptr && workspace_bytes >= w.total, TS_EWORKSPACE,
             "workspace %zu bytes < required %zu", workspace_bytes, w.total);
  TS_REQUIRE(sel_stride >= w.max_sel, TS_EWORKSPACE, "sel_stride %lld < n_init+top_k+n_local = %d",
             (long long)sel_stride, w.max_sel);
  const int max_n = bt->max_seq_len - cfg->n_init - cfg->n_local;
  TS_REQUIRE(vote_stride >= max_n, TS_EWORKSPACE, "vote_stride %lld < max candidates %d",
             (long long)vote_stride, max_n);
  TS_REQUIRE(max_n <= (1 << 20), TS_ESHAPE, "layer: at most 2^20 candidates per request (max_seq_len %d)",
             bt->max_seq_len);
  char* ws = (char*)workspace;
  // The hit flags are those the votes call left in this workspace.
  int32_t* hit = cache ? (int32_t*)(ws + w.hit) : nullptr;
  const float* ranked = votes;
  int64_t ranked_stride = vote_stride;
  if (cfg->pool_kernel > 0 && max_n > 0) {  // tr.py:366-369, after the all-reduce of tr.py:363-364
    TS_TRY(launch_pool(cfg, bt, votes, vote_stride, (float*)(ws + w.pooled), w.score_stride, hit,
                       (hipStream_t)stream));
    ranked = (const float*)(ws + w.pooled);
    ranked_stride = w.score_stride;
  }
  TopkArgs topk = make_topk_args(cfg, bt, ranked, ranked_stride, hit, cache, sel, sel_pos, sel_stride,
                                 sel_len, (uint32_t*)(ws + w.topk_ws));
  topk.clear = attn_tickets(cfg, bt->batch, w.max_sel, ws + w.attn_ws);
  topk.clear_per_req = attn_tickets_per_request(cfg);
  ts_config plain = *cfg;
  plain.pool_kernel = -1;
  if (vote_launches_planned(&plain, bt))
    topk.fault = score_votes_fault_word(&plain, bt->batch, bt->max_seq_len, ws + w.select_ws);
  TS_TRY(launch_topk(topk, bt->batch, max_n, (hipStream_t)stream));
  return launch_attn(cfg, q, k_pool, v_pool, pool_rows, sel, sel_stride, sel_len, bt->batch, w.max_sel,
                     out, ws + w.attn_ws, /*tickets_clear=*/true, (hipStream_t)stream);
}

int ts_prefill_chunk(const ts_config* cfg, const ts_batch* bt, const void* q, int32_t rows,
                     const float* cos_table, const float* sin_table, int64_t table_rows,
                     const void* k_pool, const void* v_pool, int64_t pool_rows, void* out,
                     int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                     void* workspace, size_t workspace_bytes, ts_stream_t stream) {
  TS_REQUIRE(bt != nullptr && bt->batch == 1, TS_EINVAL,
             "ts_prefill_chunk serves one request at a time (batch must be 1)");
  TS_REQUIRE(rows >= 1, TS_EINVAL, "ts_prefill_chunk: rows %d < 1", rows);
  return run_layer(cfg, bt, q, rows, cos_table, sin_table, table_rows, k_pool, v_pool, pool_rows,
                   nullptr, out, sel, sel_pos, sel_stride, sel_len, workspace, workspace_bytes,
                   stream);
}

// One chunk of the reference's extend forward in one call (tr.py:725-773): the chunk's K/V
// stored and appended (ts_kv_store_chunk), then ts_prefill_chunk.  With slots chosen by the
// caller the store rides in the chunk's first launch, the fingerprint, as spare workgroups.
int ts_prefill_step(const ts_config* cfg, const ts_batch* bt, const ts_new_kv* kv, const void* q,
                    int32_t rows, const float* cos_table, const float* sin_table, int64_t table_rows,
                    void* k_pool, void* v_pool, int64_t pool_rows, void* out, int32_t* sel,
                    int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream) {
  TS_REQUIRE(bt != nullptr && bt->batch == 1 && kv != nullptr, TS_EINVAL,
             "ts_prefill_step serves one request at a time (batch must be 1) and needs the chunk's K/V");
  TS_REQUIRE(rows >= 1, TS_EINVAL, "ts_prefill_step: rows %d < 1", rows);
  TS_REQUIRE(bt->table != nullptr && bt->seq_lens != nullptr, TS_EINVAL, "ts_prefill_step: NULL table / seq_lens");
  int32_t* table = const_cast<int32_t*>(bt->table);
  int32_t* seq_len = const_cast<int32_t*>(bt->seq_lens);
  const bool rides = kv->pages == nullptr && bt->rerun == 0 && kv->max_tokens <= 0x1fffff &&
                     rows <= 1023 * 32;
  if (!rides) {
    if (bt->rerun == 0)  // (a call that repeats a chunk after a give-up does not append again)
      TS_TRY(ts_kv_store_chunk(cfg, kv->k, kv->v, kv->out_cache_loc, kv->pages, rows, k_pool, v_pool, pool_rows,
                               table, seq_len, kv->max_tokens, stream));
    return run_layer(cfg, bt, q, rows, cos_table, sin_table, table_rows, k_pool, v_pool, pool_rows, nullptr,
                     out, sel, sel_pos, sel_stride, sel_len, workspace, workspace_bytes, stream);
  }
  // The checks ts_kv_store_chunk makes.
  TS_TRY(validate_config(cfg));
  TS_REQUIRE(kv->k && kv->v && kv->out_cache_loc && k_pool && v_pool, TS_EINVAL,
             "ts_prefill_step: NULL tensor argument");
  TS_REQUIRE_ALIGNED(kv->k, 16, "k");
  TS_REQUIRE_ALIGNED(kv->v, 16, "v");
  TS_REQUIRE_ALIGNED(k_pool, 16, "k_pool");
  TS_REQUIRE_ALIGNED(v_pool, 16, "v_pool");
  TS_REQUIRE(cfg->page_size == 1, TS_EINVAL, "ts_prefill_step: pages of %d tokens need a page pool", cfg->page_size);
  TS_REQUIRE(pool_rows >= 1 && pool_rows <= 0x7fffffffLL && kv->max_tokens >= 1, TS_EINVAL,
             "ts_prefill_step: pool_rows=%lld max_tokens=%d out of range", (long long)pool_rows, kv->max_tokens);
  ChunkStore cs{};
  cs.k = (const uint4*)kv->k;
  cs.v = (const uint4*)kv->v;
  cs.loc = kv->out_cache_loc;
  cs.k_pool = (uint4*)k_pool;
  cs.v_pool = (uint4*)v_pool;
  cs.pool_rows = pool_rows;
  cs.table = table;
  cs.seq_len = seq_len;
  cs.rows = rows;
  cs.row_vec = cfg->num_kv_heads * cfg->head_dim * 2 / 16;
  cs.max_tokens = kv->max_tokens;
  return run_layer(cfg, bt, q, rows, cos_table, sin_table, table_rows, k_pool, v_pool, pool_rows, nullptr,
                   out, sel, sel_pos, sel_stride, sel_len, workspace, workspace_bytes, stream, nullptr, &cs);
}

}  // extern "C"
