"""Oracle: chunked prefill of one request (test infrastructure only).

Follows ``patched_radix_attention_extend_forward_flashinfer``
(``patcher/token_retrieval.py:703-775``): the prompt is cut into chunks of
``PREFILL_CHUNK_SIZE`` = 512 rows (tr.py:34, 715); per chunk the chunk's K/V are
stored first (tr.py:725-733), one selection is made for the whole chunk from the
mean of its rotated queries (tr.py:735-737, 380-392), and FlashInfer's paged
prefill runs the chunk's queries over the selected slots with ``causal=True``
(tr.py:759-771).

FlashInfer (un-vendored, version not pinned, README.md:44) defines for a chunk of
``m`` query rows over ``S`` keys: query row ``i`` sits at position ``S - m + i``
and sees key ``j`` iff ``j <= S - m + i``; with ``pos_encoding_mode="ROPE_LLAMA"``
the query is rotated to that position and key ``j`` to ``j``; GQA head ``h``
reads KV head ``h // (H / Hkv)``; ``logit = sm_scale * q' . k'``, optional soft
cap, fp32 softmax, output in the query dtype.  The chunk's own tokens are the
last ``m`` entries of the selected list as long as ``n_local >= m`` (they lie inside
the local window), which is what makes the causal mask meaningful; the reference
runs any ``N_Local`` (its ``patch()`` default is 16 with 512-row chunks,
tr.py:885-894), and the alignment above then applies to whatever the list holds.
With fewer keys than rows (``S < m``) the first ``m - S`` rows see no key; FlashInfer
normalises such a row with a zero reciprocal, so its output is zero.  **Parity
unpinned** for that corner (FlashInfer is not in the tree): pinned only by the
mathematics of the mask (``tests/test_oracle.py``).
"""

from typing import List, Optional

import torch

from . import attend as _attend
from . import select as _select

PREFILL_CHUNK_SIZE = 512  # tr.py:34


def sparse_prefill_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                             slots: torch.Tensor, sm_scale: float, rope_theta: float,
                             rope_scale: float = 1.0, logit_cap: float = 0.0,
                             rope_mode: str = "ROPE_LLAMA", causal: bool = True) -> torch.Tensor:
    """``q`` [m, H, D] bf16 un-rotated, pools [P, Hkv, D] bf16, ``slots`` [S]
    physical KV slots in attention order.  Returns [m, H, D] in q's dtype; rows that see
    no key (position ``S - m + i`` negative) are zero."""
    m, num_heads, _ = q.shape
    num_kv = k_pool.shape[1]
    group = num_heads // num_kv
    idx = slots.to(torch.int64)
    s_len = idx.shape[0]
    k = k_pool[idx].float()                                # [S, Hkv, D]
    v = v_pool[idx].float()
    qf = q.float()
    q_pos = torch.arange(s_len - m, s_len)                 # [m]
    if rope_mode == "ROPE_LLAMA":
        qf = _attend._rope_llama(qf, q_pos.unsqueeze(-1).expand(m, num_heads), rope_theta, rope_scale)
        k = _attend._rope_llama(k, torch.arange(s_len).unsqueeze(-1).expand(s_len, num_kv),
                                rope_theta, rope_scale)
    elif rope_mode != "NONE":
        raise ValueError(rope_mode)
    kv_of_head = torch.arange(num_heads) // group
    logits = torch.einsum("mhd,shd->hms", qf, k[:, kv_of_head]) * sm_scale
    if logit_cap > 0:
        logits = logit_cap * torch.tanh(logits / logit_cap)
    if causal:
        visible = torch.arange(s_len).unsqueeze(0) <= q_pos.unsqueeze(1)   # [m, S]
        logits = logits.masked_fill(~visible.unsqueeze(0), float("-inf"))
        blind = ~visible.any(dim=1)                                        # [m]
        logits[:, blind] = 0.0                                             # (softmax of -inf rows is NaN)
    p = torch.softmax(logits, dim=-1)
    if causal:
        p[:, blind] = 0.0
    out = torch.einsum("hms,shd->mhd", p, v[:, kv_of_head])
    return out.to(q.dtype)


def prefill_chunk(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, tab: torch.Tensor,
                  seq_len: int, num_heads: int, head_dim: int, n_init: int, n_local: int, k: int,
                  rope_base: float, rope_scale: float, sm_scale: float, logit_cap: float = 0.0,
                  rope_mode: str = "ROPE_LLAMA", kernel_size: int = -1,
                  detail: Optional[dict] = None, qf_override: Optional[torch.Tensor] = None):
    """One chunk after its K/V have been stored: ``q`` [m, H*D] bf16 un-rotated,
    ``tab[:seq_len]`` the request's table including the chunk.  Returns
    ``(slots [S], out [m, H*D])``.  ``qf_override`` replaces the fingerprint (used to
    follow a device-computed mean, whose fp32 summation order differs)."""
    m = q.shape[0]
    slots = _select.retrieval_indices(q, k_pool, tab, seq_len, num_heads, head_dim, n_init,
                                      n_local, k, rope_base, rope_scale, kernel_size=kernel_size,
                                      detail=detail, qf_override=qf_override)
    if slots is None:                                       # tr.py:741-744
        slots = tab[:seq_len]
    out = sparse_prefill_attention(q.view(m, num_heads, head_dim), k_pool, v_pool, slots, sm_scale,
                                   rope_base, rope_scale, logit_cap, rope_mode)
    return slots, out.reshape(m, -1)


def prefill(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor, k_pool: torch.Tensor,
            v_pool: torch.Tensor, tab: torch.Tensor, seq_len: int, new_slots: torch.Tensor,
            num_heads: int, head_dim: int, n_init: int, n_local: int, k: int, rope_base: float,
            rope_scale: float, sm_scale: float, logit_cap: float = 0.0,
            rope_mode: str = "ROPE_LLAMA", chunk: int = PREFILL_CHUNK_SIZE,
            details: Optional[List[dict]] = None,
            qf_overrides: Optional[List[torch.Tensor]] = None):
    """The whole extend forward of one layer for one request: ``q`` [T, H*D],
    ``k_new`` / ``v_new`` [T, Hkv, D] written to ``new_slots`` [T] and appended to
    ``tab`` (which must have room for ``seq_len + T`` entries) chunk by chunk.
    Pools and ``tab`` are modified in place.  ``qf_overrides[i]`` replaces the
    fingerprint of chunk i (see ``prefill_chunk``).  Returns ``out`` [T, H*D]."""
    total = q.shape[0]
    outs = []
    for start in range(0, total, chunk):
        end = min(start + chunk, total)
        loc = new_slots[start:end].to(torch.int64)
        k_pool[loc] = k_new[start:end]
        v_pool[loc] = v_new[start:end]
        tab[seq_len:seq_len + (end - start)] = new_slots[start:end].to(tab.dtype)
        seq_len += end - start
        d = {} if details is not None else None
        _, o = prefill_chunk(q[start:end], k_pool, v_pool, tab, seq_len, num_heads, head_dim,
                             n_init, n_local, k, rope_base, rope_scale, sm_scale, logit_cap,
                             rope_mode, detail=d,
                             qf_override=None if qf_overrides is None else qf_overrides[start // chunk])
        if details is not None:
            details.append(d)
        outs.append(o)
    return torch.cat(outs)
