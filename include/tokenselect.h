/*
 * tokenselect.h - C ABI of libtokenselect_hip.so: TokenSelect's decode-time
 * token-level KV selection and sparse attention for AMD MI355X (gfx950).
 *
 * Every entry point takes plain pointers and sizes.  All data pointers are
 * device pointers unless a parameter says "host".  bf16 tensors are passed as
 * `const void*` (16-bit brain floats, row-major, innermost dimension
 * contiguous).  Tensors and KV pools must be aligned to 16 bytes, workspaces to
 * 256 (what hipMalloc and the framework allocators give; a view at an odd
 * offset is refused with TS_EINVAL).  Launches are asynchronous on the given HIP stream; the library
 * never synchronises and never allocates device memory.  Its only mutable
 * process-wide state is the ts_set_fused_select() switch (and the built-in
 * scratch buffer of ts_sparse_decode_attn_static); everything else lives in the
 * caller's buffers, so calls are re-entrant across streams.
 *
 * Return value: TS_OK or a negative TS_E* code; ts_last_error() then holds a
 * thread-local message.  Arguments are validated on the host before anything
 * touches the GPU, so a bad call fails without a device.
 *
 * Citations "tr.py:N" are into the reference's patcher/token_retrieval.py.
 */
#ifndef TOKENSELECT_H_
#define TOKENSELECT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TS_VERSION 100

#define TS_OK 0
#define TS_EINVAL (-1)     /* null pointer or scalar out of range            */
#define TS_ESHAPE (-2)     /* head_dim / head-group shape not supported      */
#define TS_EWORKSPACE (-3) /* workspace or an output stride is too small     */
#define TS_EHIP (-4)       /* the HIP runtime reported a launch error        */

#define TS_ROPE_NONE 0
#define TS_ROPE_LLAMA 1 /* FlashInfer pos_encoding_mode="ROPE_LLAMA", tr.py:822 */

#define TS_HEADMAP_MOD 0 /* kv head = h % Hkv: the reference's scoring, tr.py:202 */
#define TS_HEADMAP_DIV 1 /* kv head = h / (H/Hkv): conventional GQA             */

#define TS_DTYPE_F32 0
#define TS_DTYPE_BF16 1

typedef void* ts_stream_t; /* a hipStream_t; NULL is the default stream */

/* Static per-layer configuration: the module globals that patch() sets
 * (tr.py:29-39, 885-918) plus the attention scalars RadixAttention carries
 * (tr.py:816-822). */
typedef struct ts_config {
  int32_t num_heads;    /* H: query heads on this rank                        */
  int32_t num_kv_heads; /* Hkv: KV heads on this rank; H % Hkv == 0           */
  int32_t head_dim;     /* D: 128                                             */
  int32_t page_size;    /* tokens per KV page; 1 = the reference's per-token  */
                        /* table token_indices, tr.py:293-297                 */
  int32_t n_init;       /* sink tokens always kept (N_INIT)                   */
  int32_t n_local;      /* local-window tokens always kept (N_Local)          */
  int32_t top_k;        /* TOP_K; upper bound of the per-request k            */
  int32_t pool_kernel;  /* KERNEL_SIZE for vote max-pooling, <= 0 = off       */
  int32_t head_map;     /* TS_HEADMAP_* used by the scoring pass              */
  int32_t rope_mode;    /* TS_ROPE_* applied inside the attention kernel      */
  float rope_theta;     /* ROPE_BASE                                          */
  float rope_scale;     /* ROPE_SCALE                                         */
  float sm_scale;       /* RadixAttention.scaling                             */
  float logit_cap;      /* RadixAttention.logit_cap; <= 0 = off               */
} ts_config;

/* The running requests of one decode step.  The reference handles one request
 * (tr.py:130); a batch applies the same semantics to each request on its own. */
typedef struct ts_batch {
  int32_t batch;            /* B                                               */
  int32_t max_seq_len;      /* host: upper bound of seq_lens[], sizes grids    */
  const int32_t* seq_lens;  /* [B] tokens held per request, the new one included
                               (num_tokens[layer], tr.py:376)                  */
  const int32_t* table;     /* logical page -> physical page; request b's row
                               starts at table + b*table_stride.  Physical slot
                               of logical token t: table[t/ps]*ps + t%ps       */
  int64_t table_stride;     /* elements between rows                           */
  const int32_t* k_per_req; /* [B] per-request k (<= top_k), or NULL = top_k   */
  uint32_t* fault;          /* NULL, or one 32-bit word the device can write
                               (device memory, or pinned host memory that the
                               device maps, which the host may read at any time
                               without synchronising): set to 1 when a grid-wide
                               wait of a ts_select launch gave up, never cleared
                               by the library                                   */
  const int32_t* host_seq_lens; /* NULL, or [B] in host memory: upper bounds of
                               seq_lens[] that the host knows (a serving
                               framework's CPU copy of the lengths), each <=
                               max_seq_len.  Only sizes launches: a batch that
                               is too large for one ts_select launch is scored
                               and voted on in phases (as by ts_score_vote)
                               packed by these bounds instead of by
                               max_seq_len, which saves the workgroups that
                               would find no candidates (16 requests of
                               4K..128K: 439 instead of 453 us per layer).
                               The device's seq_lens[] still rule; a bound
                               below the device's value is the caller's error:
                               the tokens beyond it are not scored, and the
                               launch reports it like a wait that gave up
                               (fault, sel_len = -1)                           */
  int32_t* threshold_hint;  /* NULL, or [B] in device memory, owned by the caller and
                               kept per (request, layer) across decode steps; zero
                               before a request's first step.  ts_select leaves a
                               coarse code of where the k-th vote lay there and uses
                               the previous step's as a guess: while the votes of a
                               layer drift slowly from step to step, as the queries
                               do, the selection is then through after one meeting of
                               its workgroups instead of two (C2: 4 us of 62).  Only
                               ever a guess: a wrong or stale value costs the saving,
                               never the result, which is exact either way          */
  /* Per-call options; all zero = the defaults. */
  int32_t separate_kernels; /* 1: this call selects with ts_score + ts_vote +
                               ts_topk_ragged's kernels, whose workgroups never wait
                               for each other, whatever ts_set_fused_select says:
                               the way out for a caller whose ts_select gave up  */
  int32_t rerun;            /* 1: this call repeats the caller's previous call of
                               the same step after that one gave up (sel_len[b] =
                               -1 marks the requests concerned, and sel_len must be
                               the array of that call): the selection cache takes a
                               request that gave up as a miss whatever it cached
                               meanwhile, and its counters do not advance again  */
  uint32_t wait_us;         /* bound of a grid-wide wait of the fused kernels in
                               microseconds; 0 = TS_DEFAULT_WAIT_US              */
  int32_t absent_workgroups; /* tests of the give-up path only (0 in production):
                               workgroups counted as members of every rendezvous
                               that never arrive, so that every wait gives up
                               after wait_us while all kernels still exit        */
  int32_t workspace_clean;  /* ts_decode_layer only.  1: the caller states that this
                               workspace was last used by a ts_decode_layer call with
                               the same cfg, batch, max_seq_len and cache == NULL that
                               completed without a give-up, and by nothing since (every
                               such call leaves the selection's counters zero again:
                               its attention kernel clears them on the side).  The
                               layer then starts with the selection kernel, which
                               rotates the query itself (bit-identical to ts_rope_apply);
                               the launch that rotates and clears is not needed.  Honoured
                               where the selection is the single ts_select launch and no
                               selection cache is used; ignored otherwise.  A wrong
                               statement gives wrong selections or waits that give up */
} ts_batch;

/* Default bound of a grid-wide wait: a selection that has the device to itself
 * meets within tens of microseconds, so 10 ms means something else holds the GPU. */
#define TS_DEFAULT_WAIT_US 10000u

/* Optional selection-cache state for one layer (tr.py:301-322, 394-421).
 * All arrays are device memory owned by the caller and persist across steps. */
typedef struct ts_selcache {
  void* q_cache;        /* [B, H*D] bf16: fingerprint of the last miss          */
  int32_t* topk_cache;  /* [B, top_k] cached logical positions (+n_init)        */
  int32_t* cache_len;   /* [B] entries cached; 0 = no query seen (is_first_query) */
  int64_t* counters;    /* [B, 2] skip_count, retrieval_count (tr.py:420-421)   */
  float threshold;      /* similarity_threshold, bf16(0.9)=0.8984375 (tr.py:313) */
} ts_selcache;

/* Free pages of a paged KV pool, for the store entry points when the library and
 * not the serving framework places new tokens (any page_size; required when
 * page_size > 1).  All arrays are device memory owned by the caller.  The list is a
 * stack: entries [0, *free_count) are free and a store takes them from the top,
 * free_pages[*free_count - 1] first, for the requests that need one in request
 * order; the host returns pages by writing them at the top and raising the count
 * between launches.  ticket is one word that is zero before the first call and
 * between calls; the store kernels count their workgroups in it and reset it. */
typedef struct ts_page_pool {
  const int32_t* free_pages; /* [capacity] physical page numbers                 */
  int32_t* free_count;       /* [1]                                              */
  uint32_t* ticket;          /* [1]                                              */
} ts_page_pool;

int ts_version(void);
const char* ts_last_error(void);

/* TS_OK when the library supports this configuration (head_dim 128; Hkv in
 * {1,2,4,8}; H/Hkv from 1 to 8; power-of-two page size), else the error. */
int ts_check_config(const ts_config* cfg);

/* RotaryEmbedding.apply_rotary_pos_emb (tr.py:98-107):
 * out = bf16(float(x)*cos[pos] + float(rotate_half(x))*sin[pos]), products and
 * sum rounded separately as torch does.  x, out: [rows, heads, dim] bf16;
 * cos_table, sin_table: [table_rows, dim] fp32; position_ids: [rows] int64, or
 * NULL when every row uses table row 0. */
int ts_rope_apply(const void* x, void* out, const float* cos_table, const float* sin_table,
                  const int64_t* position_ids, int64_t table_rows, int64_t rows,
                  int32_t heads, int32_t dim, ts_stream_t stream);

/* paged_matmul (tr.py:234-261): scores[h,t] = sum_d query[h,d] *
 * token[indices[t], h % Hkv, d], fp32 accumulation, no scaling.
 * query [H,D] bf16; token [pool_rows,Hkv,D] bf16; indices [n] int32;
 * scores [H,n] of scores_dtype (the reference allocates bf16, tr.py:345-347). */
int ts_paged_matmul(const void* query, const void* token, int64_t pool_rows,
                    const int32_t* indices, void* scores, int32_t scores_dtype, int64_t n,
                    int32_t num_heads, int32_t num_kv_heads, int32_t head_dim,
                    ts_stream_t stream);

/* Scoring pass of get_topk_tokens over a ragged batch (tr.py:350-359), one
 * kernel launch: for every request that is not dense (n_init+k+n_local >= L,
 * tr.py:377) and whose skip[b] is 0, the fp32 score of every candidate t in
 * [0, L-n_init-n_local) and query head, and per-workgroup softmax partials
 * (max, sum exp) that ts_vote merges.
 * scores is tile-major so that it can be written in long bursts:
 *   scores[((b*score_stride/16 + t/16)*H + slot)*16 + t%16],
 * 16 candidates per tile, head slot = kvh*G + g for query g of KV head kvh
 * (head kvh + Hkv*g under TS_HEADMAP_MOD, head kvh*G + g under TS_HEADMAP_DIV);
 * score_stride is the number of candidate slots per request, a multiple of 16.
 * partials holds at least ts_score_partials_bytes() bytes.  qf [B,H,D] bf16 is
 * the rotated fingerprint (tr.py:380-392). */
size_t ts_score_partials_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
/* Recommended score_stride / vote_stride for max_seq_len (a multiple of 64). */
int64_t ts_score_stride(int32_t max_seq_len);
int ts_score(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
             int64_t pool_rows, const int32_t* skip, float* scores, int64_t score_stride,
             float* partials, size_t partials_bytes, ts_stream_t stream);

/* Soft vote (tr.py:361): merges the partials into stats[(b*H+h)*2 + {0,1}] =
 * {max_t s, sum_t exp(s - max)} (by head h), then votes[b*vote_stride + t] =
 * sum_h exp(s[h,t]-max_h)/Z_h from the tile-major scores, then the optional
 * max-pool of tr.py:366-369 when cfg->pool_kernel > 0 (pooled is then the result
 * and votes the scratch; both [B, vote_stride]). */
int ts_vote(const ts_config* cfg, const ts_batch* bt, const float* scores,
            int64_t score_stride, const float* partials, const int32_t* skip, float* stats,
            float* votes, float* pooled, int64_t vote_stride, ts_stream_t stream);

/* ts_score + ts_vote without the [H, n] scores in memory (tr.py:350-361): the
 * requests are served in groups ("phases") whose fp32 scores fit the LDS of the
 * device, in which the workgroups poll for each other's softmax
 * statistics (and meet once with cfg->pool_kernel > 0) and then write the votes; a batch of
 * any size is served as long as one request fits (some 260K candidates for 32
 * heads) and pool_kernel is at most 256 (ts_score_vote_supported).  The requests are
 * packed by what they can hold (ts_batch.host_seq_lens where given, max_seq_len
 * else) into phases of up to 8 consecutive requests that fit half the device (all of
 * it for a request that needs more), the workgroups of up to 24 phases in one launch,
 * which the device works through in order, so that one phase streams keys while
 * another waits for its statistics.  votes
 * [B, vote_stride] fp32 receives what ts_vote's votes (pooled with pool_kernel > 0)
 * would hold, up to the last bit of an fp32 sum taken in another order.  workspace:
 * ts_select_workspace_bytes().  The launches are ordinary ones whose workgroups must
 * be resident together, as for ts_select, with the same bounded waits; a wait that
 * gave up sets *bt->fault and the workspace's fault word (ts_select).
 * No counterpart in the reference, which materialises the scores. */
int ts_score_vote_supported(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
int ts_score_vote(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                  int64_t pool_rows, const int32_t* skip, float* votes, int64_t vote_stride,
                  void* workspace, size_t workspace_bytes, ts_stream_t stream);

/* Ragged top-k + sort + index assembly (tr.py:371-373, 433-449).  Per request:
 * the k_b largest votes (ties: lowest position first), ascending, offset by
 * n_init, between the n_init sink positions and the n_local newest positions;
 * sel_pos holds those logical positions, sel the physical slots through the
 * table, sel_len[b] = n_init+k_b+n_local.  A dense request (tr.py:377-378)
 * gets all L positions.  With hit != NULL and hit[b] != 0 the middle segment is
 * taken from cache->topk_cache instead (tr.py:419); on a miss the new positions
 * are stored there when cache != NULL (tr.py:415).
 * sel, sel_pos: [B, sel_stride] int32, sel_stride >= n_init+top_k+n_local. */
size_t ts_topk_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
int ts_topk_ragged(const ts_config* cfg, const ts_batch* bt, const float* votes,
                   int64_t vote_stride, const int32_t* hit, const ts_selcache* cache,
                   int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                   void* workspace, size_t workspace_bytes, ts_stream_t stream);

/* The whole selection in one launch (tr.py:350-373, 424-449 without the [H, n]
 * score tensor, the [n] vote vector or the sort in between): score, per-head
 * softmax, vote, exact k-th largest vote, ascending positions, index assembly.
 * The scores stay in LDS.  The softmax statistics need no meeting (the
 * per-workgroup partials and the merged statistics are polled for: the data
 * is its own flag); the workgroups of the launch then meet two to four times:
 * histogram rounds over the 11 + 11 + 10 bits of the vote keys until at most 256 candidates are left around the k-th
 * vote, which are listed and ranked by every workgroup in a last round together
 * with the per-workgroup counts that place its selected positions in the output
 * (masses of exact ties take all three histogram rounds and a count round; one
 * more round with cfg->pool_kernel > 0: the max-pool of tr.py:366-369 needs the
 * votes of the neighbouring workgroups).  Outputs and the hit / cache arguments are those of
 * ts_topk_ragged (same tie rule: lowest position first); votes, when not NULL,
 * also receives the [B, vote_stride] fp32 votes (pooled when pool_kernel > 0).
 * Usable when ts_select_supported() returns 1: pool_kernel at most 256 and batch x
 * candidates small enough (some 260K candidates for 32 heads) for the scores to
 * fit the LDS of the device; TS_ESHAPE otherwise, and the caller runs
 * ts_score + ts_vote + ts_topk_ragged.  The launch is an ordinary one sized so
 * that all its workgroups are resident together; that holds while nothing else
 * runs on the device beside the caller's stream (a cooperative launch would
 * enforce it, at about 25 us per call).  Every grid-wide wait is bounded (bt->wait_us,
 * 10 ms unless the caller says otherwise);
 * once one has given up the others return at once, the kernel drains, and the
 * launch reports it without any host synchronisation: sel_len[b] = -1 for
 * every request that was selecting (the other outputs of those requests are
 * not valid; ts_sparse_decode_attn treats a negative length as an empty list),
 * *bt->fault = 1 when bt->fault is given, and the first 32-bit word of the
 * last batch * 65 * 4096 bytes of the workspace is 1 until the next clearing.  A
 * caller that sees it reruns the step with the separate kernels (bt->separate_kernels).
 * No counterpart in the reference, which materialises every intermediate. */
int ts_select_supported(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
size_t ts_select_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
int ts_select(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
              int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
              int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
              int64_t vote_stride, void* workspace, size_t workspace_bytes, ts_stream_t stream);
/* ts_select is two launches: a small kernel that clears the counters and rendezvous
 * words in the workspace, and the selection kernel.  A caller that has another
 * kernel of its own clear them (ts_decode_layer folds the clearing into its rotation
 * kernel), or that wants to time the selection kernel alone, makes the two calls
 * itself: ts_select_clear() once before every ts_select_cleared() on the same
 * workspace, for the same cfg, batch and max_seq_len.  Same arguments, results and
 * errors as ts_select.  No counterpart in the reference. */
int ts_select_clear(const ts_config* cfg, const ts_batch* bt, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream);
int ts_select_cleared(const ts_config* cfg, const ts_batch* bt, const void* qf, const void* k_pool,
                      int64_t pool_rows, const int32_t* hit, const ts_selcache* cache, int32_t* sel,
                      int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, float* votes,
                      int64_t vote_stride, void* workspace, size_t workspace_bytes,
                      ts_stream_t stream);

/* ts_select_cleared with an explicit bound for the grid-wide waits, in ticks of
 * the device's 100 MHz clock (ts_select uses bt->wait_us x 100, by default 1 000 000 = 10 ms;
 * these arguments take the place of bt->wait_us and bt->absent_workgroups), and a number of
 * workgroups that are counted as members of the rendezvous but never arrive
 * (0 in production): with absent_workgroups > 0 every wait gives up after
 * wait_ticks, which is how the give-up path is tested without hanging a GPU.
 * No counterpart in the reference. */
int ts_select_cleared_bounded(const ts_config* cfg, const ts_batch* bt, const void* qf,
                              const void* k_pool, int64_t pool_rows, const int32_t* hit,
                              const ts_selcache* cache, int32_t* sel, int32_t* sel_pos,
                              int64_t sel_stride, int32_t* sel_len, float* votes,
                              int64_t vote_stride, void* workspace, size_t workspace_bytes,
                              uint64_t wait_ticks, int32_t absent_workgroups, ts_stream_t stream);

/* Selection-cache decision (tr.py:394-401, 416-421) for one layer, no host
 * sync: hit[b] = cache_len[b] > 0 && cos(q_cache[b], qf[b]) >= threshold; on a
 * miss q_cache[b] = qf[b].  Dense requests (tr.py:377) are left untouched with
 * hit[b] = 0.  Counters advance as the reference's do. */
int ts_selcache_step(const ts_config* cfg, const ts_batch* bt, const void* qf,
                     const ts_selcache* cache, int32_t* hit, ts_stream_t stream);

/* Decode attention over the selected slots: FlashInfer
 * BatchDecodeWithPagedKVCacheWrapper.forward with page_size 1 as called at
 * tr.py:815-823.  Head h reads KV head h/(H/Hkv); with TS_ROPE_LLAMA the query
 * is rotated to position S-1 and selected key j to position j inside the kernel.
 * q, out: [B,H,D] bf16; k_pool, v_pool: [pool_rows,Hkv,D] bf16;
 * sel [B, sel_stride] int32 with sel_len[b] valid entries (<= max_sel_len); every
 * row holds at least max_sel_len entries, those past sel_len[b] are read (the
 * slots are requested together with the length) but not used.
 * The products run on the matrix cores (v_mfma_f32_16x16x32_bf16, fp32 accumulation) with
 * every fp32 operand - rotated key, rotated query, softmax weight - split into two bf16
 * halves, so that the result equals an fp32 evaluation to the rounding of the bf16 output. */
size_t ts_attn_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_sel_len);
int ts_sparse_decode_attn(const ts_config* cfg, const void* q, const void* k_pool,
                          const void* v_pool, int64_t pool_rows, const int32_t* sel,
                          int64_t sel_stride, const int32_t* sel_len, int32_t batch,
                          int32_t max_sel_len, void* out, void* workspace,
                          size_t workspace_bytes, ts_stream_t stream);

/* ts_sparse_decode_attn for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid hipMalloc): same
 * arguments, kernels and results, but the split-K partials and tickets live in a
 * buffer built into the library (ts_attn_static_scratch_bytes() = 4 MiB of device
 * memory per GPU the library runs on, held until the process ends) instead of a
 * caller's workspace.  The call allocates and frees nothing.  TS_EWORKSPACE when
 * batch x heads x splits needs more than the buffer holds (about 7900 partial rows
 * of 520 bytes; with 32 query / 8 KV heads: every batch up to 251).  All calls on one GPU share the buffer:
 * calls that overlap on one GPU (two streams, two threads) race and must be
 * serialised by the caller; calls on one stream are ordered by the stream.
 * ts_attn_static_scratch_bytes() also looks up the buffer of the current device (as
 * the first call on a device would): make it once per device at set-up, before any
 * capture begins.  No counterpart in the reference. */
size_t ts_attn_static_scratch_bytes(void);
int ts_sparse_decode_attn_static(const ts_config* cfg, const void* q, const void* k_pool,
                                 const void* v_pool, int64_t pool_rows, const int32_t* sel,
                                 int64_t sel_stride, const int32_t* sel_len, int32_t batch,
                                 int32_t max_sel_len, void* out, ts_stream_t stream);

/* KV store + table append (patched_radix_attention_store_kv_cache tr.py:844-854,
 * add_k_cache tr.py:332-336).
 * pages == NULL, page_size 1 (the reference): the framework has chosen the slots,
 *   k_pool[loc[b]] = k[b], v_pool[loc[b]] = v[b], table[b][seq_lens[b]] = loc[b],
 *   seq_lens[b] += 1.
 * pages != NULL (any page_size; out_cache_loc is not read): the new token of request
 *   b, at position L = seq_lens[b], goes to slot table[b][L/ps]*ps + L%ps; when
 *   L % ps == 0 the request first takes a fresh page from the pool (in request
 *   order, top of the stack first) and table[b][L/ps] receives it.  A request
 *   whose table is full (L >= max_tokens) or that finds no page left is left
 *   untouched; *free_count drops by the pages taken.
 * k, v: [batch, Hkv, D] bf16; table rows hold ceil(max_tokens / ps) entries. */
int ts_kv_store(const ts_config* cfg, const void* k, const void* v, const int32_t* out_cache_loc,
                const ts_page_pool* pages, void* k_pool, void* v_pool, int64_t pool_rows,
                int32_t* table, int64_t table_stride, int32_t* seq_lens, int32_t batch,
                int32_t max_tokens, ts_stream_t stream);

/* The reference's decode forward of a layer in one call
 * (patched_radix_attention_decode_forward_flashinfer, tr.py:777-825): the new token's
 * K/V stored and appended as ts_kv_store does it (kv: its k, v, out_cache_loc, pages
 * and max_tokens; the table and the lengths are bt's, which the call therefore
 * writes), then ts_decode_layer on the lengths after the append (bt->max_seq_len and
 * host_seq_lens bound those).  Results are those of the two calls.  With a selection
 * cache the store rides in the layer's first launch, the rotation and cache decision
 * (slots chosen by the caller or taken from a page pool alike), and a step is three
 * kernels instead of four; otherwise the two calls follow each other.  With
 * bt->rerun the step's token has been appended by the call that gave up, and only
 * the layer runs. */
typedef struct ts_new_kv {
  const void* k;                 /* [batch, Hkv, D] bf16 */
  const void* v;
  const int32_t* out_cache_loc;  /* [batch] slots, or NULL with pages */
  const ts_page_pool* pages;     /* or NULL */
  int32_t max_tokens;            /* as for ts_kv_store */
} ts_new_kv;
int ts_decode_step(const ts_config* cfg, const ts_batch* bt, const ts_new_kv* kv, const void* q,
                   const float* q_cos, const float* q_sin, void* k_pool, void* v_pool,
                   int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                   int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                   size_t workspace_bytes, ts_stream_t stream);

/* The QKV projection of a decode step with the KV store as its epilogue: what the
 * serving stack does in two places, qkv = x W^T (+ bias) in the model's attention
 * module and then patched_radix_attention_store_kv_cache (tr.py:844-854) +
 * add_k_cache (tr.py:332-336), in one pass over W.  Columns [0, H*D) of the product
 * go to q_out [batch, H*D]; the next Hkv*D to k_pool[loc[b]], the last Hkv*D to
 * v_pool[loc[b]]; then table[b][seq_lens[b]] = loc[b], seq_lens[b] += 1 as
 * ts_kv_store does, with the caller's slots (pages == NULL, page_size 1; a full
 * table leaves table and length alone) or with slots from the table / the page
 * pool (pages != NULL, as for ts_kv_store).  x: [batch, hidden]
 * bf16; w: [(H + 2 Hkv) * D, hidden] bf16 row-major (torch Linear weight);
 * bias: [(H + 2 Hkv) * D] bf16 or NULL; fp32 accumulation, bf16 outputs.
 * batch <= 8 and hidden a multiple of 8, at most 4096 (TS_ESHAPE otherwise: use a
 * library GEMM and ts_kv_store). */
int ts_qkv_store(const ts_config* cfg, const void* x, const void* w, const void* bias,
                 int32_t hidden, const int32_t* out_cache_loc, const ts_page_pool* pages,
                 void* q_out, void* k_pool,
                 void* v_pool, int64_t pool_rows, int32_t* table, int64_t table_stride,
                 int32_t* seq_lens, int32_t batch, int32_t max_tokens, ts_stream_t stream);

/* ---- chunked prefill (patched_radix_attention_extend_forward_flashinfer,
 * tr.py:703-775): per chunk of at most 512 rows of one request the chunk's K/V
 * are stored, one selection is made from the mean of the chunk's rotated
 * queries, and the chunk attends causally over the selected slots. ---- */

/* store_kv_cache(start, end) + add_k_cache for a chunk (tr.py:725-733,
 * 332-336).  pages == NULL, page size 1: k_pool[loc[r]] = k[r], v likewise,
 * table[*seq_len + r] = loc[r] for r < rows, then *seq_len += rows (one
 * launch for rows <= 8184 and max_tokens < 2^21: the upper bits of *seq_len
 * count the workgroups while the kernel runs, and are zero again when it ends).
 * pages != NULL: row r goes to position *seq_len + r of the paged table, the
 * request's last page first and then fresh pages from the top of the pool, in
 * order; one launch.
 * k, v: [rows, Hkv, D] bf16; table: the request's row; rows beyond max_tokens
 * (or beyond the pages left) are dropped. */
int ts_kv_store_chunk(const ts_config* cfg, const void* k, const void* v,
                      const int32_t* out_cache_loc, const ts_page_pool* pages, int32_t rows,
                      void* k_pool, void* v_pool,
                      int64_t pool_rows, int32_t* table, int32_t* seq_len, int32_t max_tokens,
                      ts_stream_t stream);

/* Fingerprint of a chunk (tr.py:380-392): row i of q [rows, H, D] bf16 rotated
 * with rows n_local + i of the [table_rows, D] fp32 cos / sin tables, rounded
 * to bf16 (bit-identical to ts_rope_apply), then the mean over the rows, in
 * fp32, rounded to bf16: qf [H, D]. */
int ts_fingerprint(const ts_config* cfg, const void* q, int32_t rows, const float* cos_table,
                   const float* sin_table, int64_t table_rows, void* qf, ts_stream_t stream);

/* FlashInfer paged prefill over the selected slots with causal=True
 * (tr.py:759-771), page size 1, one request: query row i of q [rows, H, D] sits
 * at position S - rows + i (S = *sel_len <= max_sel_len), is rotated
 * to it, and attends to the keys sel[j], rotated to j, for j <= S - rows + i
 * (FlashInfer's alignment of the last query row with the last key; with fewer keys
 * than rows the first rows - S rows see no key and their output is zero);
 * GQA head h reads KV head h / (H/Hkv); sm_scale, logit_cap as in
 * ts_sparse_decode_attn.  out: [rows, H, D] bf16.  The workspace receives the
 * selected keys, rotated, and the selected values, transposed, once per call
 * (2 * Hkv * max_sel_len * D bf16, rounded up). */
size_t ts_prefill_attn_workspace_bytes(const ts_config* cfg, int32_t max_sel_len);
int ts_sparse_prefill_attn(const ts_config* cfg, const void* q, int32_t rows, const void* k_pool,
                           const void* v_pool, int64_t pool_rows, const int32_t* sel,
                           const int32_t* sel_len, int32_t max_sel_len, void* out, void* workspace,
                           size_t workspace_bytes, ts_stream_t stream);

/* One chunk of the extend forward after its KV store (tr.py:735-773):
 * fingerprint -> selection -> causal sparse attention, for the single request
 * of bt (batch 1; seq_lens[0] already counts the chunk).  While rows <= n_local the
 * chunk's own tokens are the tail of the selected list; a longer chunk is served as
 * the reference serves it (tr.py:716-738 with any N_Local): the list ends with the
 * last n_local tokens, the chunk's earlier rows are candidates like any other token,
 * and row i still sees the list's entries j <= S - rows + i.  Workspace as
 * for ts_decode_layer (ts_decode_layer_workspace_bytes(cfg, 1, max_seq_len)).
 * q, out: [rows, H*D] bf16. */
int ts_prefill_chunk(const ts_config* cfg, const ts_batch* bt, const void* q, int32_t rows,
                     const float* cos_table, const float* sin_table, int64_t table_rows,
                     const void* k_pool, const void* v_pool, int64_t pool_rows, void* out,
                     int32_t* sel, int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len,
                     void* workspace, size_t workspace_bytes, ts_stream_t stream);

/* One chunk of the extend forward in one call (tr.py:725-773): ts_kv_store_chunk of the
 * chunk's K/V (kv: k, v [rows, Hkv, D], out_cache_loc [rows], pages, max_tokens; the
 * table row and the length word are bt's, which the call therefore writes), then
 * ts_prefill_chunk on the length after the append (which bt->max_seq_len bounds).
 * Results are those of the two calls.  With slots chosen by the caller (pages == NULL,
 * page_size 1) the store rides in the chunk's first launch, the fingerprint, as spare
 * workgroups; otherwise the two calls follow each other.  With bt->rerun the chunk has been
 * appended by the call that gave up, and only ts_prefill_chunk runs. */
int ts_prefill_step(const ts_config* cfg, const ts_batch* bt, const ts_new_kv* kv, const void* q,
                    int32_t rows, const float* cos_table, const float* sin_table, int64_t table_rows,
                    void* k_pool, void* v_pool, int64_t pool_rows, void* out, int32_t* sel,
                    int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream);

/* One layer of patched_radix_attention_decode_forward_flashinfer after the KV
 * store (tr.py:791-825): fingerprint (q rotated with q_cos/q_sin, the [D] table
 * rows of position n_local, tr.py:380-388) -> [selection cache] -> score ->
 * vote -> top-k -> assembly -> sparse attention.  q, out: [B,H*D] bf16.
 * cache may be NULL (QUERY_CACHE=False as released, tr.py:918).
 *
 * When ts_select_supported() holds, the selection runs as the single ts_select
 * kernel; a batch too large for that (many requests, or contexts so long that each
 * request needs the device to itself) is scored and voted on as by ts_score_vote, in
 * one launch as a rule, and then ranked by the kernels of ts_topk_ragged; where
 * neither serves (pool_kernel above 256, a request that does not fit the device)
 * ts_score, ts_vote and ts_topk_ragged run as they do on their own.  All forms give
 * the same selection.
 * ts_set_fused_select(0) forces the separate kernels for the calling process
 * (1 restores the default); it returns the previous setting and has no
 * counterpart in the reference. */
int ts_set_fused_select(int enable);
/* Which form ts_decode_layer takes for a shape: 2 = ts_select, 1 = ts_score_vote's
 * launch + top-k kernels, 0 = ts_score + ts_vote + top-k kernels; -1 for an
 * unsupported configuration.  The second form answers for a batch descriptor (the
 * same answer: host_seq_lens changes how the phases are packed, not the form). */
int ts_decode_layer_selection(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
int ts_decode_layer_selection_of(const ts_config* cfg, const ts_batch* bt);
size_t ts_decode_layer_workspace_bytes(const ts_config* cfg, int32_t batch, int32_t max_seq_len);
int ts_decode_layer(const ts_config* cfg, const ts_batch* bt, const void* q, const float* q_cos,
                    const float* q_sin, const void* k_pool, const void* v_pool,
                    int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                    int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                    size_t workspace_bytes, ts_stream_t stream);

/* ts_decode_layer split at the vote, for tensor parallelism (tr.py:361-364: every rank
 * scores its own heads, the ranks add up their partial votes with one all-reduce, and
 * all then select the same tokens): ts_decode_layer_votes runs fingerprint ->
 * [selection cache] -> score -> per-head softmax -> sum over this rank's heads and
 * leaves the un-pooled votes in votes [B, vote_stride] fp32 (requests that are dense
 * or hit the cache are not written); the caller adds the ranks' votes in place (an
 * all-reduce(SUM) over xGMI; nothing to do on one rank); ts_decode_layer_attend runs
 * [max-pool, tr.py:366-369] -> top-k -> assembly -> sparse attention over this rank's
 * heads.  Both calls take the same cfg (this rank's num_heads / num_kv_heads), batch,
 * cache and workspace (ts_decode_layer_workspace_bytes; the hit flags of the cache
 * travel in it).  On one rank the two calls give what ts_decode_layer gives.
 * The selection cache compares this rank's slice of the query, so ranks may disagree
 * on a hit: use it with one rank only. */
int ts_decode_layer_votes(const ts_config* cfg, const ts_batch* bt, const void* q, const float* q_cos,
                          const float* q_sin, const void* k_pool, int64_t pool_rows,
                          const ts_selcache* cache, float* votes, int64_t vote_stride,
                          void* workspace, size_t workspace_bytes, ts_stream_t stream);
int ts_decode_layer_attend(const ts_config* cfg, const ts_batch* bt, const void* q, const float* votes,
                           int64_t vote_stride, const void* k_pool, const void* v_pool,
                           int64_t pool_rows, const ts_selcache* cache, void* out, int32_t* sel,
                           int32_t* sel_pos, int64_t sel_stride, int32_t* sel_len, void* workspace,
                           size_t workspace_bytes, ts_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TOKENSELECT_H_ */
