"""Oracle: the selection cache (test infrastructure only).

Restates the *intended* behaviour of the ``QUERY_CACHE`` branch of
``patcher/token_retrieval.py:394-421`` with its state from tr.py:301-322.  The
reference ships that branch switched off (tr.py:918) and it cannot run as
written (wrong arity at tr.py:412; ``cosine_similarity`` on 1-D inputs with the
default ``dim``), so there is nothing executable to compare with: parity unpinned.

Semantics per (request, layer):

* miss when no query has been cached yet or ``cos(q_cached, q_now) < thr``
  (tr.py:395-401); ``thr`` is 0.9 stored in bf16, i.e. 0.8984375 (tr.py:313-315);
* on a miss the selection runs, and both the selected positions (already
  offset by ``n_init``) and the query fingerprint are cached (tr.py:411-417) -
  the anchor is the query of the last miss, not the previous step's query;
* on a hit the cached positions are reused and ``skip_count`` grows (tr.py:419-420);
* ``retrieval_count`` grows on every call (tr.py:421);
* the sink and local-window segments are always rebuilt from the current
  length (tr.py:436-446).
"""

from typing import Callable

import torch

THRESHOLD = float(torch.tensor(0.9, dtype=torch.bfloat16))  # 0.8984375


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a64, b64 = a.double(), b.double()
    return float((a64 @ b64) / max(float(a64.norm() * b64.norm()), 1e-8))


class SelectionCache:
    def __init__(self, threshold: float = THRESHOLD, anchor: str = "last_miss"):
        assert anchor in ("last_miss", "previous")
        self.threshold = threshold
        self.anchor = anchor
        self.q_cached = None
        self.top_cached = None
        self.skip_count = 0
        self.retrieval_count = 0

    def step(self, qf: torch.Tensor, select: Callable[[], torch.Tensor]):
        """Returns ``(top_pos, hit)``; ``select()`` yields positions incl. ``+n_init``."""
        miss = self.q_cached is None or cosine(self.q_cached, qf) < self.threshold
        if miss:
            top = select()
            self.top_cached = top.clone()
            self.q_cached = qf.clone()
        else:
            top = self.top_cached
            self.skip_count += 1
            if self.anchor == "previous":      # non-reference variant, for contrast tests
                self.q_cached = qf.clone()
        self.retrieval_count += 1
        return top, not miss
