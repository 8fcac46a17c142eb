"""CPU oracle for the TokenSelect decode hot path.

TEST INFRASTRUCTURE ONLY.  This package is a PyTorch-on-CPU restatement of the
reference algorithm (``/root/reference/patcher/token_retrieval.py`` plus the
FlashInfer paged-decode semantics the reference calls into).  It is the parity
checker for the HIP kernels and the CPU baseline that ``bench.py`` times.
Nothing in ``tokenselect_amd`` may import it: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.

What pins each function (no reference test, golden vector or fixture exists for
this path, and the reference module itself needs SGLang / vLLM / FlashInfer /
a CUDA GPU, none of which are available):

* ``rope``      - independent complex-multiplication formulation, identity at
                  position 0, norm preservation, relative-position property.
* ``score``     - ``torch.einsum`` on the gathered rows, one-hot known answers,
                  brute-force Python loops, ``%``-vs-``//`` head-map discriminator.
* ``vote``      - ``torch.softmax(...).sum(0)``, mass invariant, shift invariance.
* ``topk``      - ``torch.argsort`` on tie-free inputs, planted known answers.
* ``assemble``  - structural invariants (prefix / suffix / length / identity table).
* ``attend``    - ``F.scaled_dot_product_attention`` with RoPE disabled, full
                  selection == textbook attention, position-shift invariance.
* ``prefill``   - causal attention against ``F.scaled_dot_product_attention`` with
                  an explicit mask (RoPE off), a one-row chunk == ``attend``, row
                  ``i`` == decode attention over the first ``S - m + i + 1`` keys.
* ``store``     - the per-token append is a slice assignment (tr.py:332-336); the
                  paged append (no reference counterpart: an extension, like
                  batches) is pinned by what the page arithmetic fixes: a chunk
                  equals the same tokens appended one by one, slots equal the
                  expanded page table, pages taken = ceil((L+m)/ps) - ceil(L/ps),
                  a page size of 1 reduces to popping one slot per token.
* ``selcache``  - pure-Python replay of the state machine.  The reference ships
                  this branch disabled and not runnable (tr.py:918, 412, 397), so
                  its behaviour is *intended* semantics: parity unpinned.

Parity unpinned (absorbed by the stated tolerances, cannot be checked here):
the bf16 rounding / reduction order of Triton 3.0.0's ``tl.sum`` on NVIDIA, the
tie order of CUDA ``torch.topk``, and FlashInfer's ``__sincosf`` error.
"""

from . import rope, select, attend, selcache, layer, prefill, store  # noqa: F401
