"""A Llama-shaped decoder whose attention is the TokenSelect decode layer: the
caller either side of the hot path, as the serving stack drives it
(``RadixAttention.forward`` -> ``patched_radix_attention_forward`` tr.py:827-842:
store the new token's K/V and append it to the token table, tr.py:844-854,
332-336, then select and attend, tr.py:777-825) on every layer of the model.

Only the attention goes through the library; the projections, norms and the MLP
are torch's library GEMMs and elementwise kernels.  The model applies no rotary
embedding of its own: keys are cached un-rotated and both the scoring query and
the attention rotate inside the library (tr.py:381-392, 822).

The KV cache is laid out as the reference's: one ``[rows, Hkv, D]`` K pool and V
pool per layer, slot ids shared by all layers, a per-request table of slots per
logical position (page size 1, tr.py:293-297) and a token count per layer and
request (``num_tokens[layer]``, tr.py:298).
"""

from dataclasses import dataclass
from typing import List, Optional, Sequence

import torch
import torch.nn.functional as F

from . import ops
from .ops import Batch, DecodeLayer, LayerConfig, SelectionCache


@dataclass
class ModelConfig:
    """Llama-3-8B by default."""
    layers: int = 32
    hidden: int = 4096
    intermediate: int = 14336
    vocab: int = 128256
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rms_eps: float = 1e-5
    rope_theta: float = 5e5
    init_std: float = 0.02
    n_init: int = 128
    n_local: int = 512
    top_k: int = 4096

    def layer_config(self) -> LayerConfig:
        return LayerConfig(num_heads=self.num_heads, num_kv_heads=self.num_kv_heads,
                           head_dim=self.head_dim, page_size=1, n_init=self.n_init,
                           n_local=self.n_local, top_k=self.top_k, rope_theta=self.rope_theta)


def _normal_bf16(shape, std: float, gen, device) -> torch.Tensor:
    """N(0, std) in bf16, drawn in slabs so that no fp32 copy of a large tensor exists."""
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(-1)
    slab = 1 << 28
    for lo in range(0, flat.numel(), slab):
        flat[lo:lo + slab].normal_(0.0, std, generator=gen)
    return out


class Decoder:
    """Random-initialised decoder with a prefilled random KV cache.

    ``contexts[b]`` tokens of request b are already cached (N(0,1) keys and
    values, slots drawn from a random permutation); ``new_tokens`` more can be
    decoded.  ``query_cache`` switches the selection cache on (one per layer,
    tr.py:301-322); the reference serves with it off (tr.py:897).  ``fused_qkv``
    (default: where the shape allows) runs the QKV projection with the KV store as
    its epilogue instead of a library GEMM followed by ``ts_kv_store``."""

    def __init__(self, mc: ModelConfig, contexts: Sequence[int], new_tokens: int, device,
                 seed: int = 0, query_cache: bool = False, fused_qkv: Optional[bool] = None):
        self.mc, self.cfg, self.device = mc, mc.layer_config(), device
        self.contexts, self.new_tokens = list(contexts), new_tokens
        B = self.batch = len(self.contexts)
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)
        hd, kvd = mc.num_heads * mc.head_dim, mc.num_kv_heads * mc.head_dim
        std = mc.init_std
        self.embed = _normal_bf16((mc.vocab, mc.hidden), std, gen, device)
        self.lm_head = _normal_bf16((mc.vocab, mc.hidden), std, gen, device)
        self.final_norm = torch.ones(mc.hidden, dtype=torch.bfloat16, device=device)
        self.wqkv = [_normal_bf16((hd + 2 * kvd, mc.hidden), std, gen, device) for _ in range(mc.layers)]
        self.wo = [_normal_bf16((mc.hidden, hd), std, gen, device) for _ in range(mc.layers)]
        self.w_gate_up = [_normal_bf16((2 * mc.intermediate, mc.hidden), std, gen, device)
                          for _ in range(mc.layers)]
        self.w_down = [_normal_bf16((mc.hidden, mc.intermediate), std, gen, device)
                       for _ in range(mc.layers)]
        self.norm_in = [torch.ones(mc.hidden, dtype=torch.bfloat16, device=device)
                        for _ in range(mc.layers)]
        self.norm_post = [torch.ones(mc.hidden, dtype=torch.bfloat16, device=device)
                          for _ in range(mc.layers)]

        # KV cache: every request owns contexts[b] + new_tokens slots of the permutation.
        self.max_len = max(self.contexts) + new_tokens
        rows = sum(self.contexts) + B * new_tokens
        order = torch.randperm(rows, generator=gen, device=device).to(torch.int32)
        self.table = torch.zeros((B, self.max_len), dtype=torch.int32, device=device)
        self.free = torch.empty((new_tokens, B), dtype=torch.int32, device=device)
        at = 0
        for b, L in enumerate(self.contexts):
            self.table[b, :L] = order[at:at + L]
            self.free[:, b] = order[at + L:at + L + new_tokens]
            at += L + new_tokens
        self.k_pools = [_normal_bf16((rows, mc.num_kv_heads, mc.head_dim), 1.0, gen, device)
                        for _ in range(mc.layers)]
        self.v_pools = [_normal_bf16((rows, mc.num_kv_heads, mc.head_dim), 1.0, gen, device)
                        for _ in range(mc.layers)]
        self.num_tokens = torch.tensor(self.contexts, dtype=torch.int32, device=device) \
            .repeat(mc.layers, 1).contiguous()
        self.decoded = 0
        # QKV projection + KV store in one kernel where the library serves the shape.
        supported = ops.qkv_store_supported(B, mc.hidden)
        self.fused_qkv = supported if fused_qkv is None else (fused_qkv and supported)
        self.attention = DecodeLayer(self.cfg, B, self.max_len, device)
        self.caches: List[Optional[SelectionCache]] = [
            SelectionCache.allocate(self.cfg, B, device) if query_cache else None
            for _ in range(mc.layers)]
        # Per (layer, request): where the k-th vote of the last selection lay, the single-launch
        # selection's guess for the next step.
        self.hints = torch.zeros((mc.layers, B), dtype=torch.int32, device=device)
        # Per-call options handed to the layer (tests force a give-up through them).
        self.layer_options = {}
        self.steps_redone = 0

    def _norm(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        return F.rms_norm(x, (self.mc.hidden,), w, self.mc.rms_eps)

    @torch.no_grad()
    def decode_step(self, tokens: torch.Tensor, trace: Optional[list] = None) -> torch.Tensor:
        """One forward over ``tokens`` [B] (the last token of every request): stores
        their K/V, attends through the TokenSelect layer, returns the logits
        ``[B, vocab]`` (bf16).  ``trace`` receives, per layer, clones of the query, key and
        value rows, the attention output, the selected slots and their count."""
        mc, cfg = self.mc, self.cfg
        if self.decoded >= self.new_tokens:
            raise RuntimeError("the KV cache has no slot left for another token")
        loc = self.free[self.decoded]
        max_len = max(self.contexts) + self.decoded + 1
        # The lengths after this step's store, on the host too (a serving stack has them
        # there): the layer then packs its scoring phases by what the requests hold.
        host_lens = torch.tensor([c + self.decoded + 1 for c in self.contexts], dtype=torch.int32)
        hd, kvd = mc.num_heads * mc.head_dim, mc.num_kv_heads * mc.head_dim
        x = self.embed[tokens]
        for l in range(mc.layers):
            h = self._norm(x, self.norm_in[l])
            if self.fused_qkv:  # projection with the KV store as its epilogue
                q = ops.qkv_store(cfg, h, self.wqkv[l], None, loc, self.k_pools[l], self.v_pools[l],
                                  self.table, self.num_tokens[l])
                k = v = None
            else:
                q, k, v = F.linear(h, self.wqkv[l]).split((hd, kvd, kvd), dim=-1)
                q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
            bt = Batch(self.num_tokens[l], self.table, max_len, host_seq_lens=host_lens, hint=self.hints[l],
                       **self.layer_options)
            if k is None:
                attn, sel, _, sel_len = self.attention(q, self.k_pools[l], self.v_pools[l], bt, self.caches[l])
            else:  # the store and the layer in one call, as the reference's decode forward has them
                attn, sel, _, sel_len = self.attention.step(q, k, v, loc, self.k_pools[l], self.v_pools[l], bt,
                                                            self.caches[l])
            if trace is not None:
                if k is None:   # the rows as they landed in the pools
                    k = self.k_pools[l][loc.long()].reshape(self.batch, kvd)
                    v = self.v_pools[l][loc.long()].reshape(self.batch, kvd)
                trace.append((q.clone(), k.clone(), v.clone(), attn.clone(), sel.clone(), sel_len.clone()))
            x = x + F.linear(attn, self.wo[l])
            gate, up = F.linear(self._norm(x, self.norm_post[l]), self.w_gate_up[l]).chunk(2, dim=-1)
            x = x + F.linear(F.silu(gate) * up, self.w_down[l])
        self.decoded += 1
        return F.linear(self._norm(x, self.final_norm), self.lm_head)

    @torch.no_grad()
    def decode_step_checked(self, tokens: torch.Tensor):
        """:meth:`decode_step` the way a serving loop runs it: the next tokens are read
        back to the host, and at that synchronisation point a fused selection kernel that
        gave up anywhere in the step is noticed.  The step is then undone (the token
        counts go back by one; the slots, and so the stored K/V, are the same when it
        runs again; selection-cache entries, which the failed launch may have half
        written, are dropped, so the requests select afresh) and repeated with the
        separate kernels, which the model keeps from then on.  Returns ``(logits, next
        tokens on the device, next tokens on the host)``."""
        before = self.decoded
        try:
            logits = self.decode_step(tokens)
            nxt = logits.argmax(dim=-1)
            host = nxt.cpu()
            failed = self.attention.gave_up()
        except ops.SelectionGaveUp:  # a later layer's call saw the word before the step ended
            torch.cuda.current_stream().synchronize()
            failed = True
        if failed:
            self.attention._latch()
            self.decoded = before
            lens = torch.tensor([c + before for c in self.contexts], dtype=torch.int32)
            self.num_tokens.copy_(lens.repeat(self.mc.layers, 1))
            for cache in self.caches:
                if cache is not None:
                    cache.cache_len.zero_()
            self.layer_options = {k: v for k, v in self.layer_options.items()
                                  if k not in ("absent_workgroups", "wait_us")}
            self.steps_redone += 1
            logits = self.decode_step(tokens)
            nxt = logits.argmax(dim=-1)
            host = nxt.cpu()
        return logits, nxt, host

    @torch.no_grad()
    def generate(self, tokens: torch.Tensor, steps: int, read_back: bool = False) -> torch.Tensor:
        """Greedy decoding: ``[steps, B]`` token ids.  Without ``read_back`` there is no
        host synchronisation inside, and a selection that gave up is reported when the
        loop ends (SelectionGaveUp: the tokens are not valid); with it every step's tokens
        go to the host as a server's would, and a step that gave up is redone there."""
        out = torch.empty((steps, self.batch), dtype=torch.int64, device=self.device)
        for t in range(steps):
            if read_back:
                tokens = self.decode_step_checked(tokens)[1]
            else:
                tokens = self.decode_step(tokens).argmax(dim=-1)
            out[t] = tokens
        if not read_back:
            torch.cuda.current_stream().synchronize()
            self.attention.check()
        return out
