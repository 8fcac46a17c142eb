"""Oracle: KV store and token-table append (test infrastructure only).

The reference appends one table entry per stored token,
``token_indices[layer, num_tokens : num_tokens + len(indices)] = indices``
(``patcher/token_retrieval.py:332-336``), after scattering the K / V rows to the
slots the serving framework chose (tr.py:844-854).  That is ``append_slots``.

With pages of more than one token the table holds one entry per page and the
slot of logical position ``t`` is ``table[t // ps] * ps + t % ps``
(``select.expand_page_table``).  The reference has no such mode; the paged append
restated here is the per-token rule carried over: a request whose length is a
multiple of the page size takes a fresh page, the requests of one step in request
order, each from the top of a stack of free pages.
"""

from typing import List, Optional

import torch


def append_slots(table_row: torch.Tensor, seq_len: int, slots: torch.Tensor, max_tokens: int) -> int:
    """tr.py:332-336 for one layer: entries that do not fit are dropped.  Returns the new length."""
    fit = max(min(int(slots.shape[0]), max_tokens - seq_len), 0)
    table_row[seq_len:seq_len + fit] = slots[:fit].to(table_row.dtype)
    return seq_len + fit


def append_token_paged(table: torch.Tensor, seq_lens: List[int], free_pages: List[int],
                       page_size: int, max_tokens: int, pool_rows: int) -> List[Optional[int]]:
    """One decode step for a batch: ``table`` [B, pages] and ``seq_lens`` / ``free_pages``
    (a stack, last element = top) are modified in place.  Returns the slot of every
    request's new token, ``None`` where the table was full or no page was left."""
    count = len(free_pages)
    plans, rank = [], 0
    for b, L in enumerate(seq_lens):                     # the plan, from the state before the step
        if not 0 <= L < max_tokens:
            plans.append(None)
            continue
        if L % page_size == 0:
            page = free_pages[count - 1 - rank] if rank < count else None
            rank += 1
            fresh = True
        else:
            page, fresh = int(table[b, L // page_size]), False
        slot = None if page is None else page * page_size + L % page_size
        if slot is not None and not 0 <= slot < pool_rows:
            slot = None
        plans.append(None if slot is None else (page, fresh, slot))
    taken = min(rank, count)
    out = []
    for b, plan in enumerate(plans):                     # the commit
        if plan is None:
            out.append(None)
            continue
        page, fresh, slot = plan
        if fresh:
            table[b, seq_lens[b] // page_size] = page
        seq_lens[b] += 1
        out.append(slot)
    del free_pages[count - taken:]
    return out


def append_chunk_paged(table_row: torch.Tensor, seq_len: int, rows: int, free_pages: List[int],
                       page_size: int, max_tokens: int):
    """A prefill chunk of one request: positions ``seq_len .. seq_len + rows - 1`` fill the
    last page and then fresh pages from the top of the stack, in order.  Rows beyond
    ``max_tokens`` or beyond the pages left are dropped.  Returns ``(slots, new_len)``."""
    slots = []
    for r in range(rows):
        L = seq_len + r
        if L >= max_tokens:
            break
        if L % page_size == 0:
            if not free_pages:
                break
            table_row[L // page_size] = free_pages.pop()
        slots.append(int(table_row[L // page_size]) * page_size + L % page_size)
    return slots, seq_len + len(slots)
