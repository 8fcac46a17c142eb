// Paged append of new tokens to the requests' tables (add_k_cache tr.py:332-336 for
// pages of more than one token): position L of request b lives in physical slot
// table[b][L / ps] * ps + L % ps; when L % ps == 0 the request takes a fresh page from
// the caller's free list.  The reference keeps one table entry per token and lets the
// serving framework pick every slot; with pages the library picks them, so that a
// decode step needs no host-side allocation.
//
// All workgroups of a store kernel derive the same plan from a snapshot that none of
// them modifies: the lengths, the table and the free count as they were at launch.
// The requests that need a page are ranked in request order and request r-th in rank
// takes free_pages[count - 1 - r] (the list is a stack, its top is taken first), so
// the assignment does not depend on the order in which workgroups run.  The workgroup
// that draws the last ticket of the launch then writes the new table entries, the new
// lengths and the new free count, and resets the ticket word for the next launch.
#pragma once

#include "ts_common.h"

namespace ts {

struct PagePool {
  const int32_t* free_pages;  // NULL: no pool (page size 1, slots given by the caller)
  int32_t* free_count;
  uint32_t* ticket;
};

static inline PagePool page_pool_of(const ts_page_pool* p) {
  PagePool pool{nullptr, nullptr, nullptr};
  if (p) {
    pool.free_pages = p->free_pages;
    pool.free_count = p->free_count;
    pool.ticket = p->ticket;
  }
  return pool;
}

// Where the new token of a request goes.
struct AppendPlan {
  bool ok;        // the table has room and, where needed, a page was left
  bool new_page;  // table[page_index] = page is to be written
  int len;        // length before the append
  int page_index;
  int32_t page;
  uint32_t slot;
};

__device__ __forceinline__ AppendPlan make_append_plan(const int32_t* table_row, int len, bool room,
                                                       bool need, uint32_t rank, int count,
                                                       const int32_t* free_pages, int page_shift,
                                                       int page_mask, uint32_t pool_rows) {
  AppendPlan p;
  p.len = len;
  p.new_page = need;
  p.page_index = len >> page_shift;
  p.ok = room && (!need || (int)rank < count);
  p.page = 0;
  if (p.ok) p.page = need ? free_pages[count - 1 - (int)rank] : table_row[p.page_index];
  const uint32_t slot = ((uint32_t)p.page << page_shift) + (uint32_t)(len & page_mask);
  p.slot = slot < pool_rows ? slot : pool_rows - 1;
  if (p.page < 0 || slot >= pool_rows) p.ok = false;
  return p;
}

// One whole wavefront walks the requests in order (64 per round, the rank of the requests
// that need a page carried from round to round); f(b, plan) sees every request's plan.
// Returns the number of pages the launch takes from the list: one per request that needed
// one while the list lasted, the top `taken` entries, so that the stack stays contiguous.
// An entry that is no page of the pool (negative, or beyond pool_rows) is taken like the
// others and dropped: its request is left untouched this step and finds the next entry at
// the next one, instead of meeting the same entry for ever.
template <typename F>
__device__ __forceinline__ int for_each_append(const int32_t* seq_lens, const int32_t* table,
                                               int64_t table_stride, int batch, const PagePool& pool,
                                               int page_shift, int max_tokens, uint32_t pool_rows,
                                               int lane, F&& f) {
  const int page_mask = (1 << page_shift) - 1;
  const int count = max(*pool.free_count, 0);
  uint32_t run = 0;
  for (int base = 0; base < batch; base += 64) {
    const int b = base + lane;
    const int len = b < batch ? seq_lens[b] : 0;
    const bool room = b < batch && len >= 0 && len < max_tokens;
    const bool need = room && (len & page_mask) == 0;
    const uint64_t mask = __ballot(need);
    const uint32_t rank = run + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
    if (b < batch)
      f(b, make_append_plan(table + (int64_t)b * table_stride, len, room, need, rank, count,
                            pool.free_pages, page_shift, page_mask, pool_rows));
    run += (uint32_t)__popcll(mask);
  }
  return min((int)run, count);
}

// The launch's last workgroup (by ticket) commits the plan: table entries, lengths,
// free count; then the ticket word is zero again.  Called by one whole wavefront of
// every workgroup after its own stores are on their way; `workgroups` = gridDim of
// the launch.
__device__ __forceinline__ void commit_appends(int32_t* seq_lens, int32_t* table, int64_t table_stride,
                                               int batch, const PagePool& pool, int page_shift,
                                               int max_tokens, uint32_t pool_rows, int lane,
                                               uint32_t workgroups) {
  uint32_t last = 0;
  if (lane == 0)
    last = __hip_atomic_fetch_add(pool.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 ==
                   workgroups
               ? 1u
               : 0u;
  if (!__shfl((int)last, 0)) return;
  const int taken = for_each_append(seq_lens, table, table_stride, batch, pool, page_shift, max_tokens,
                                    pool_rows, lane, [&](int b, const AppendPlan& p) {
                                      if (!p.ok) return;
                                      if (p.new_page) table[(int64_t)b * table_stride + p.page_index] = p.page;
                                      seq_lens[b] = p.len + 1;
                                    });
  if (lane == 0) {
    *pool.free_count = max(*pool.free_count, 0) - taken;
    __hip_atomic_store(pool.ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace ts
