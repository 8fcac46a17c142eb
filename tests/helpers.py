"""Shared helpers of the parity tests: run the oracle on a workload's tensors."""

import torch

import oracle
from tokenselect_amd.workloads import Workload


def say(*args):
    print(*args, flush=True)


def cpu_tabs(wl: Workload):
    table = wl.table.cpu()
    return [oracle.select.expand_page_table(table[b], L, wl.cfg.page_size)
            for b, L in enumerate(wl.seq_lens)]


def oracle_layer(wl: Workload, details=None):
    c = wl.cfg
    return oracle.layer.decode_layer(
        wl.q.cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), cpu_tabs(wl), wl.seq_lens, c.num_heads,
        c.head_dim, c.n_init, c.n_local, wl.k_list, c.rope_theta, c.rope_scale,
        c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5, c.logit_cap, c.rope_mode,
        c.pool_kernel, details)


def assert_attention_close(wl: Workload, b: int, out_b, slots_b, ref_slots_b, ref_out_b, what: str,
                           tol: float = 2e-2):
    """Attention output of request `b` within `tol` (absolute, bf16) of the oracle's.
    Where the device's slot list differs from the oracle's (a tie at the k-th vote
    resolved the other way), the oracle attends over the device's own slots, so that
    the output is compared in every case."""
    c = wl.cfg
    slots_b, ref_slots_b = slots_b.cpu(), ref_slots_b.cpu()
    if not torch.equal(slots_b.long(), ref_slots_b.long()):
        sm = c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5
        ref_out_b = oracle.attend.sparse_decode_attention(
            wl.q.cpu().view(len(wl.seq_lens), c.num_heads, c.head_dim)[b], wl.k_pool.cpu(),
            wl.v_pool.cpu(), slots_b, sm, c.rope_theta, c.rope_scale, c.logit_cap, c.rope_mode)
    err = (out_b.cpu().float().reshape(-1) - ref_out_b.float().reshape(-1)).abs().max().item()
    assert err <= tol, f"{what}: attention max abs err {err} > {tol}"
    return err


def assert_scores_close(got: torch.Tensor, ref: torch.Tensor, what: str, rel: float = 1e-5):
    """fp32 scores within `rel` of the oracle, measured against the score scale
    (its RMS), since individual scores pass through zero.  The stated bar is 1e-3;
    products of bf16 pairs are exact in fp32, so a correct kernel differs from the
    oracle by the order of its fp32 additions only and the tests hold it to 1e-5."""
    scale = ref.double().pow(2).mean().sqrt().item()
    err = (got.double() - ref.double()).abs().max().item()
    assert err <= rel * scale, f"{what}: max |err| {err:.3e} > {rel} * rms {scale:.3e}"
    return err / scale


def assert_index_sets_match(got_pos, ref_pos, votes_ref, n_init: int, what: str, rtol: float = 1e-5):
    """Selected positions identical except for members whose oracle vote lies
    within `rtol` (relative) of the k-th largest oracle vote."""
    got, ref = set(got_pos.tolist()), set(ref_pos.tolist())
    assert len(got) == len(got_pos), f"{what}: duplicate positions"
    if got == ref:
        return 0
    kth = votes_ref[torch.tensor(sorted(ref)) - n_init].min().item()
    for p in got ^ ref:
        v = votes_ref[p - n_init].item()
        assert abs(v - kth) <= rtol * abs(kth), (
            f"{what}: position {p} (vote {v:.9e}) differs and is not tied with the "
            f"k-th vote {kth:.9e}")
    return len(got ^ ref)
