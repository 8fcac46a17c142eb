"""Oracle: criticality scoring, soft vote, top-k and index assembly
(test infrastructure only).

Follows ``patcher/token_retrieval.py``: gather-dot tr.py:166-231, softmax + head
sum tr.py:361, max-pool smoothing tr.py:366-369, top-k + sort tr.py:371-373,
the short-context fallback and index assembly tr.py:375-449, and the
logical->physical token table tr.py:324-336.

Numerics: exact bf16 products accumulated in fp32, fp32 scores, fp32 softmax and
vote.  (The reference as released rounds the scores, the softmax and the head sum to
bf16, tr.py:345-347, 361, in an order its Triton version fixes; that chain is not
restated here.)
"""

from typing import Optional

import torch

from . import rope as _rope

_CHUNK = 8192


def expand_page_table(page_table: torch.Tensor, seq_len: int, page_size: int) -> torch.Tensor:
    """Logical position -> physical KV slot for a paged cache:
    ``slot(t) = page_table[t // page_size] * page_size + t % page_size``.
    With ``page_size == 1`` this is the reference's ``token_indices`` row
    (tr.py:293-297, 332-336)."""
    t = torch.arange(seq_len, dtype=torch.int64)
    pages = page_table.to(torch.int64)[t // page_size]
    return (pages * page_size + t % page_size).to(torch.int32)


def score(qf: torch.Tensor, k_pool: torch.Tensor, cand_slots: torch.Tensor,
          head_map: str = "mod") -> torch.Tensor:
    """``scores[h, t] = sum_d qf[h, d] * K[cand[t], kv(h), d]`` with no scaling
    (tr.py:216-224).  ``kv(h) = h % Hkv`` in the reference (tr.py:202);
    ``head_map="div"`` gives the conventional ``h // (H/Hkv)`` for comparison.

    ``qf`` is ``[H, D]`` bf16, ``k_pool`` ``[P, Hkv, D]`` bf16, ``cand_slots``
    ``[n]`` integer.  Returns ``[H, n]`` fp32.
    """
    num_heads, _ = qf.shape
    num_kv = k_pool.shape[1]
    heads = torch.arange(num_heads)
    kv_of_head = heads % num_kv if head_map == "mod" else heads // (num_heads // num_kv)
    n = cand_slots.shape[0]
    out = torch.empty((num_heads, n), dtype=torch.float32)
    slots = cand_slots.to(torch.int64)
    for lo in range(0, n, _CHUNK):
        rows = k_pool[slots[lo:lo + _CHUNK]]            # [c, Hkv, D]
        per_head = rows[:, kv_of_head]                   # [c, H, D]
        out[:, lo:lo + _CHUNK] = torch.einsum("hd,chd->hc", qf.float(), per_head.float())
    return out


def vote(scores: torch.Tensor) -> torch.Tensor:
    """Per-head softmax over the candidates, summed over heads (tr.py:361).
    fp32 in, fp32 out."""
    return torch.softmax(scores, dim=-1).sum(dim=0)


def max_pool(votes: torch.Tensor, kernel_size: int) -> torch.Tensor:
    """Sliding-window maximum applied when ``kernel_size > 0`` (tr.py:366-369):
    stride 1, padding ``(kernel_size-1)//2`` (an even kernel shortens the
    output by one element)."""
    if kernel_size <= 0:
        return votes
    return torch.nn.functional.max_pool1d(
        votes.unsqueeze(0), kernel_size=kernel_size,
        padding=(kernel_size - 1) // 2, stride=1).squeeze(0)


def topk_sorted(votes: torch.Tensor, k: int) -> torch.Tensor:
    """Positions of the ``k`` largest votes in ascending order (tr.py:371-372)."""
    idx = torch.topk(votes, k, dim=-1).indices
    return torch.sort(idx).values


def get_topk_tokens(qf: torch.Tensor, k_pool: torch.Tensor, k: int,
                    cand_slots: torch.Tensor, head_dim: int,
                    kernel_size: int = -1, return_all: bool = False):
    """tr.py:338-373 for one request: score -> vote -> [pool] -> top-k -> sort.
    ``qf`` is the flat ``[H*D]`` fingerprint."""
    s = score(qf.view(-1, head_dim), k_pool, cand_slots)
    c = max_pool(vote(s), kernel_size)
    top = topk_sorted(c, k)
    if return_all:
        return top, s, c
    return top


def assemble(tab: torch.Tensor, seq_len: int, n_init: int, n_local: int,
             top_pos: torch.Tensor) -> torch.Tensor:
    """``tab[ [0..n_init) ++ top_pos ++ [L-n_local..L) ]`` (tr.py:436-449).
    ``top_pos`` already carries the ``+ n_init`` offset (tr.py:433)."""
    pos = torch.cat([torch.arange(0, n_init), top_pos.to(torch.int64),
                     torch.arange(seq_len - n_local, seq_len)])
    return tab[pos]


def is_dense(seq_len: int, n_init: int, n_local: int, k: int) -> bool:
    """Short-context rule: the reference returns ``None`` and attends densely
    exactly when ``n_init + k + n_local >= L`` (tr.py:376-378, 793)."""
    return n_init + k + n_local >= seq_len


def retrieval_indices(q: torch.Tensor, k_pool: torch.Tensor, tab: torch.Tensor,
                      seq_len: int, num_heads: int, head_dim: int, n_init: int,
                      n_local: int, k: int, rope_base: float, rope_scale=1.0,
                      kernel_size: int = -1,
                      detail: Optional[dict] = None,
                      qf_override: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """tr.py:375-449 for one request with the selection cache disabled, as
    released (tr.py:918).  ``q`` is ``[rows, H*D]`` bf16 un-rotated, ``tab`` the
    request's logical->physical table with the new token already appended
    (store precedes select, tr.py:787-791).  Returns physical slots ``[S]`` int32
    or ``None`` for the dense fallback.  ``qf_override`` ([H*D] bf16) stands in for
    the fingerprint, for checks downstream of a fingerprint computed elsewhere."""
    if is_dense(seq_len, n_init, n_local, k):
        return None
    qf = _rope.scoring_query(q, num_heads, head_dim, n_local, rope_base, rope_scale)
    if qf_override is not None:
        qf = qf_override.reshape(-1).to(qf.dtype)
    cand = tab[n_init:seq_len - n_local]
    top, s, c = get_topk_tokens(qf, k_pool, k, cand, head_dim, kernel_size,
                                return_all=True)
    top = top + n_init
    if detail is not None:
        detail.update(qf=qf, scores=s, votes=c, top_pos=top)
    return assemble(tab, seq_len, n_init, n_local, top)
