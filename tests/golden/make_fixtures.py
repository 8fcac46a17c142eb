"""Writes ``tests/golden/decode_layer_small.npz`` and
``tests/golden/prefill_small.npz``: seeded inputs of one small decode layer and of
one small chunked prefill, and the outputs of the CPU oracle (``oracle/``) for them.

The reference holds no golden vectors for this path and cannot be imported, so
these fixtures come from this repository's own oracle; they lock the oracle
against drift and give the HIP path a fixed known-answer case.  bf16 tensors
are stored as their int16 bit patterns.

    python tests/golden/make_fixtures.py
"""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "decode_layer_small.npz")

H, HKV, D = 8, 2, 128
N_INIT, N_LOCAL, TOP_K = 4, 8, 16
PAGE = 4
ROPE_BASE = 1e4
SEQ_LENS = [120, 26, 77]      # the second request is dense (4 + 16 + 8 >= 26)


def bits(t):
    return t.view(torch.int16).numpy()


def main():
    g = torch.Generator().manual_seed(2024)
    pages_per = [-(-L // PAGE) for L in SEQ_LENS]
    total_pages = sum(pages_per)
    order = torch.randperm(total_pages, generator=g)
    table = torch.zeros((len(SEQ_LENS), max(pages_per)), dtype=torch.int32)
    at = 0
    for b, n in enumerate(pages_per):
        table[b, :n] = order[at:at + n].int()
        at += n
    rows = total_pages * PAGE
    k_pool = torch.randn(rows, HKV, D, generator=g).bfloat16()
    v_pool = torch.randn(rows, HKV, D, generator=g).bfloat16()
    q = torch.randn(len(SEQ_LENS), H * D, generator=g).bfloat16()
    tabs = [oracle.select.expand_page_table(table[b], L, PAGE) for b, L in enumerate(SEQ_LENS)]
    details = []
    sels, out = oracle.layer.decode_layer(q, k_pool, v_pool, tabs, SEQ_LENS, H, D, N_INIT, N_LOCAL,
                                          [TOP_K] * len(SEQ_LENS), ROPE_BASE, 1.0, D ** -0.5,
                                          details=details)
    arrays = dict(
        meta=np.array([H, HKV, D, N_INIT, N_LOCAL, TOP_K, PAGE], dtype=np.int64),
        rope_base=np.array([ROPE_BASE]), seq_lens=np.array(SEQ_LENS, dtype=np.int32),
        table=table.numpy(), k_pool=bits(k_pool), v_pool=bits(v_pool), q=bits(q), out=bits(out))
    for b, sel in enumerate(sels):
        arrays[f"sel_{b}"] = sel.numpy()
        if details[b]:
            arrays[f"qf_{b}"] = bits(details[b]["qf"])
            arrays[f"scores_{b}"] = details[b]["scores"].numpy()
            arrays[f"votes_{b}"] = details[b]["votes"].numpy()
            arrays[f"top_pos_{b}"] = details[b]["top_pos"].numpy()
    np.savez_compressed(OUT, **arrays)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


PREFILL_OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "prefill_small.npz")


def prefill():
    """A 70-row extend on top of 90 cached tokens, chunks of 32 rows (n_local 32)."""
    g = torch.Generator().manual_seed(2025)
    heads, kv, L0, T, chunk, n_init, n_local, top_k = 8, 2, 90, 70, 32, 4, 32, 12
    rows = L0 + T
    k_pool = torch.randn(rows, kv, D, generator=g).bfloat16()
    v_pool = torch.randn(rows, kv, D, generator=g).bfloat16()
    order = torch.randperm(rows, generator=g).int()
    tab = torch.zeros(rows, dtype=torch.int32)
    tab[:L0] = order[:L0]
    new_slots = order[L0:]
    q = torch.randn(T, heads * D, generator=g).bfloat16()
    k_new = torch.randn(T, kv, D, generator=g).bfloat16()
    v_new = torch.randn(T, kv, D, generator=g).bfloat16()
    k0, v0 = k_pool.clone(), v_pool.clone()
    details = []
    out = oracle.prefill.prefill(q, k_new, v_new, k_pool, v_pool, tab, L0, new_slots, heads, D, n_init,
                                 n_local, top_k, ROPE_BASE, 1.0, D ** -0.5, chunk=chunk,
                                 details=details)
    arrays = dict(
        meta=np.array([heads, kv, D, n_init, n_local, top_k, L0, T, chunk], dtype=np.int64),
        rope_base=np.array([ROPE_BASE]), k_pool=bits(k0), v_pool=bits(v0), table=tab[:L0].numpy(),
        new_slots=new_slots.numpy(), q=bits(q), k_new=bits(k_new), v_new=bits(v_new), out=bits(out))
    for i, d in enumerate(details):
        arrays[f"qf_{i}"] = bits(d["qf"])
        arrays[f"top_pos_{i}"] = d["top_pos"].numpy()
        arrays[f"votes_{i}"] = d["votes"].numpy()
    np.savez_compressed(PREFILL_OUT, **arrays)
    print("wrote", PREFILL_OUT, os.path.getsize(PREFILL_OUT), "bytes")


if __name__ == "__main__":
    main()
    prefill()
