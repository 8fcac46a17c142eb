"""Oracle: decode attention over the selected KV tokens (test infrastructure only).

The reference calls FlashInfer's ``BatchDecodeWithPagedKVCacheWrapper.forward``
with page size 1 on the selected slots (``patcher/token_retrieval.py:794-823``).
FlashInfer is an un-vendored dependency (``flashinfer-python``, version not
pinned, README.md:44), so its published decode algorithm is restated here:

* GQA: query head ``h`` reads KV head ``h // (H / Hkv)``.
* ``pos_encoding_mode="ROPE_LLAMA"``: rotate-half RoPE applied inside the kernel
  in fp32, query at position ``S - 1``, key ``j`` at position ``j`` (its index in
  the selected list), frequency ``(1 / rope_scale) * theta^(-2 (i mod D/2) / D)``.
* ``logit = sm_scale * q' . k'``; optional soft cap ``cap * tanh(logit / cap)``
  when ``logits_soft_cap > 0``; fp32 softmax; ``o = p @ V``; output in q's dtype.
"""

import torch


def _rope_llama(x: torch.Tensor, pos: torch.Tensor, theta: float, rope_scale: float):
    """x [..., D] fp32, pos broadcastable to x[..., 0]; rotate-half convention."""
    d = x.shape[-1]
    half = d // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = (1.0 / rope_scale) * torch.pow(torch.tensor(theta, dtype=torch.float64), -2.0 * i / d)
    ang = pos.to(torch.float64).unsqueeze(-1) * freq
    c, s = ang.cos().float(), ang.sin().float()
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def sparse_decode_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            slots: torch.Tensor, sm_scale: float, rope_theta: float,
                            rope_scale: float = 1.0, logit_cap: float = 0.0,
                            rope_mode: str = "ROPE_LLAMA") -> torch.Tensor:
    """One request.  ``q`` [H, D] bf16 un-rotated, pools [P, Hkv, D] bf16,
    ``slots`` [S] physical KV slots in attention order.  Returns [H, D] in
    ``q.dtype``."""
    num_heads, _ = q.shape
    num_kv = k_pool.shape[1]
    group = num_heads // num_kv
    idx = slots.to(torch.int64)
    s_len = idx.shape[0]
    k = k_pool[idx].float()                                # [S, Hkv, D]
    v = v_pool[idx].float()
    qf = q.float()
    if rope_mode == "ROPE_LLAMA":
        qf = _rope_llama(qf, torch.full((num_heads,), s_len - 1), rope_theta, rope_scale)
        k = _rope_llama(k, torch.arange(s_len).unsqueeze(-1).expand(s_len, num_kv),
                        rope_theta, rope_scale)
    elif rope_mode != "NONE":
        raise ValueError(rope_mode)
    kv_of_head = torch.arange(num_heads) // group
    logits = torch.einsum("hd,shd->hs", qf, k[:, kv_of_head]) * sm_scale
    if logit_cap > 0:
        logits = logit_cap * torch.tanh(logits / logit_cap)
    p = torch.softmax(logits, dim=-1)
    out = torch.einsum("hs,shd->hd", p, v[:, kv_of_head])
    return out.to(q.dtype)
