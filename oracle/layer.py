"""Oracle: one decode step of one layer for a batch of independent requests
(test infrastructure only).

The reference serves a single running request (``patcher/token_retrieval.py:130``);
a batch is defined as the single-request semantics applied to every request on
its own: store precedes select precedes attend (tr.py:787-823), a short context
attends densely over ``tab[0:L]`` (tr.py:377-378, 741-744).
"""

from typing import List, Optional

import torch

from . import attend as _attend
from . import select as _select


def decode_layer(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                 tabs: List[torch.Tensor], seq_lens: List[int], num_heads: int,
                 head_dim: int, n_init: int, n_local: int, ks: List[int],
                 rope_base: float, rope_scale: float, sm_scale: float,
                 logit_cap: float = 0.0, rope_mode: str = "ROPE_LLAMA",
                 kernel_size: int = -1, details: Optional[list] = None):
    """``q`` [B, H*D] bf16 un-rotated.  ``tabs[b]`` is request b's
    logical->physical table (at least ``seq_lens[b]`` long).  Returns
    ``(slots_per_request, out [B, H*D])``."""
    outs, sels = [], []
    for b, (tab, seq_len, k) in enumerate(zip(tabs, seq_lens, ks)):
        d = {} if details is not None else None
        slots = _select.retrieval_indices(q[b:b + 1], k_pool, tab, seq_len, num_heads,
                                          head_dim, n_init, n_local, k, rope_base,
                                          rope_scale, kernel_size=kernel_size, detail=d)
        if slots is None:
            slots = tab[:seq_len]
        if details is not None:
            details.append(d)
        o = _attend.sparse_decode_attention(q[b].view(num_heads, head_dim), k_pool, v_pool,
                                            slots, sm_scale, rope_base, rope_scale,
                                            logit_cap, rope_mode)
        sels.append(slots)
        outs.append(o.reshape(-1))
    return sels, torch.stack(outs)
