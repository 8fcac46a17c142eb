"""Seeded synthetic decode workloads: a paged KV pool, per-request page tables,
queries and the layer configuration.  Used by the benchmark and the parity
tests; tensors are generated on the requested device from a ``torch.Generator``
seeded per workload, so CPU and GPU runs of the same seed differ in values but
not in shape or statistics.

Shapes follow the two model families the reference ships configs for
(``config/llama-token-retrieval.yaml``, ``config/qwen-token-retrieval.yaml``):
``n_init`` 128, ``n_local`` 512, ``top_k`` 2048, rope base 5e5 / 1e6.
"""

from dataclasses import dataclass, field
from typing import List, Optional

import torch

from .ops import Batch, LayerConfig

LLAMA3_8B = dict(num_heads=32, num_kv_heads=8, rope_theta=5e5)
QWEN2_7B = dict(num_heads=28, num_kv_heads=4, rope_theta=1e6)


@dataclass
class Workload:
    name: str
    cfg: LayerConfig
    q: torch.Tensor          # [B, H*D] bf16, un-rotated
    k_pool: torch.Tensor     # [P, Hkv, D] bf16
    v_pool: torch.Tensor
    table: torch.Tensor      # [B, pages] int32
    seq_lens: List[int]
    seq_lens_dev: torch.Tensor
    k_list: List[int]
    k_per_req: Optional[torch.Tensor] = None
    planted: List[torch.Tensor] = field(default_factory=list)  # per request: logical positions
    free_pages: Optional[torch.Tensor] = None   # [extra_pages] int32: pages no request holds
    host_lengths: bool = False                  # hand the lengths to the library on the host too
    hint: Optional[torch.Tensor] = None         # [B] int32: Batch.hint, kept across the steps of a run

    @property
    def batch(self) -> Batch:
        host = torch.tensor(self.seq_lens, dtype=torch.int32) if self.host_lengths else None
        return Batch(self.seq_lens_dev, self.table, max(self.seq_lens), self.k_per_req,
                     host_seq_lens=host, hint=self.hint)

    def score_bytes(self) -> int:
        """Algorithmic bytes of the scoring pass: every candidate K row once,
        the table entries that locate them, and the queries."""
        c = self.cfg
        row = c.num_kv_heads * c.head_dim * 2
        total = 0
        for L, k in zip(self.seq_lens, self.k_list):
            if c.n_init + k + c.n_local >= L:
                continue
            n = L - c.n_init - c.n_local
            total += n * row + (-(-L // c.page_size)) * 4
        return total + len(self.seq_lens) * c.num_heads * c.head_dim * 2

    def attn_bytes(self) -> int:
        c = self.cfg
        row = c.num_kv_heads * c.head_dim * 2
        total = 0
        for L, k in zip(self.seq_lens, self.k_list):
            s = L if c.n_init + k + c.n_local >= L else c.n_init + k + c.n_local
            total += s * (2 * row + 4)
        return total + 2 * len(self.seq_lens) * c.num_heads * c.head_dim * 2


def _randn_bf16(shape, gen, device, chunk_rows: int = 1 << 18) -> torch.Tensor:
    out = torch.empty(shape, dtype=torch.bfloat16, device=device)
    flat = out.view(shape[0], -1)
    for lo in range(0, shape[0], chunk_rows):
        hi = min(shape[0], lo + chunk_rows)
        flat[lo:hi] = torch.randn((hi - lo, flat.shape[1]), generator=gen, device=device,
                                  dtype=torch.float32).to(torch.bfloat16)
    return out


def _rotated_query(q: torch.Tensor, cfg: LayerConfig) -> torch.Tensor:
    """fp32 rotate-half RoPE of q [B, H, D] at position n_local (planting only)."""
    d = cfg.head_dim
    inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, d, 2, dtype=torch.float32, device=q.device) / d))
    ang = cfg.n_local * cfg.rope_scale * inv
    c, s = torch.cat((ang, ang)).cos(), torch.cat((ang, ang)).sin()
    x = q.float()
    rot = torch.cat((-x[..., d // 2:], x[..., :d // 2]), dim=-1)
    return x * c + rot * s


def build(name: str, shape: dict, seq_lens: List[int], k_list: List[int], page_size: int,
          device, seed: int, permute_pages: bool = True, plant_frac: float = 0.0,
          plant_sigma: float = 3.0, n_init: int = 128, n_local: int = 512,
          top_k: Optional[int] = None, extra_pages: int = 0, pool_kernel: int = -1) -> Workload:
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    cfg = LayerConfig(num_heads=shape["num_heads"], num_kv_heads=shape["num_kv_heads"],
                      page_size=page_size, n_init=n_init, n_local=n_local,
                      top_k=top_k if top_k is not None else max(k_list),
                      rope_theta=shape["rope_theta"], rope_scale=1.0, pool_kernel=pool_kernel)
    B = len(seq_lens)
    pages_per_req = [-(-L // page_size) for L in seq_lens]
    total_pages = sum(pages_per_req) + extra_pages
    order = (torch.randperm(total_pages, generator=gen, device=device) if permute_pages
             else torch.arange(total_pages, device=device))
    table = torch.zeros((B, max(pages_per_req)), dtype=torch.int32, device=device)
    at = 0
    for b, n_pages in enumerate(pages_per_req):
        table[b, :n_pages] = order[at:at + n_pages].to(torch.int32)
        at += n_pages
    rows = total_pages * page_size
    k_pool = _randn_bf16((rows, cfg.num_kv_heads, cfg.head_dim), gen, device)
    v_pool = _randn_bf16((rows, cfg.num_kv_heads, cfg.head_dim), gen, device)
    q = torch.randn((B, cfg.num_heads * cfg.head_dim), generator=gen, device=device,
                    dtype=torch.float32).to(torch.bfloat16)

    planted = []
    if plant_frac > 0:
        qr = _rotated_query(q.view(B, cfg.num_heads, cfg.head_dim), cfg)
        for b, L in enumerate(seq_lens):
            n = L - n_init - n_local
            count = max(1, int(round(plant_frac * n)))
            pos = torch.randperm(n, generator=gen, device=device)[:count].sort().values + n_init
            pages = table[b, (pos // page_size).long()].long()
            slots = pages * page_size + pos % page_size
            for kvh in range(cfg.num_kv_heads):  # heads mapped to kvh by h % Hkv
                mean_q = qr[b, kvh::cfg.num_kv_heads].mean(0)
                unit = mean_q / mean_q.norm()
                k_pool[slots, kvh] = (k_pool[slots, kvh].float() + plant_sigma * unit).to(torch.bfloat16)
            planted.append(pos)

    seq_dev = torch.tensor(seq_lens, dtype=torch.int32, device=device)
    k_dev = None
    if any(k != cfg.top_k for k in k_list):
        k_dev = torch.tensor(k_list, dtype=torch.int32, device=device)
    return Workload(name, cfg, q, k_pool, v_pool, table, list(seq_lens), seq_dev, list(k_list),
                    k_dev, planted, order[at:].to(torch.int32).contiguous())


def config1(device, seed: int = 0, seq_len: int = 32768, top_k: int = 2048) -> Workload:
    """Qwen2-7B layer, one request, per-token table (page size 1), permuted."""
    return build("C1 qwen2-7b B1 L%d k%d page1" % (seq_len, top_k), QWEN2_7B, [seq_len], [top_k], 1,
                 device, seed)


def config2(device, seed: int = 1, seq_len: int = 131072, top_k: int = 2048) -> Workload:
    """Llama-3-8B layer, one request, page size 16 with a permuted page table;
    1 % of the candidates carry a +3 sigma shift along the query direction."""
    return build("C2 llama3-8b B1 L%d k%d page16" % (seq_len, top_k), LLAMA3_8B, [seq_len], [top_k],
                 16, device, seed, plant_frac=0.01)


def config3(device, seed: int = 2, batch: int = 16, lo: int = 4096, hi: int = 131072,
            top_k: int = 2048) -> Workload:
    """Ragged batch sharing one pool: L_b ~ U{lo..hi}, k_b = min(top_k, L_b/4)."""
    gen = torch.Generator()
    gen.manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (batch,), generator=gen).tolist()
    ks = [min(top_k, L // 4) for L in lens]
    return build("C3 llama3-8b B%d ragged page16" % batch, LLAMA3_8B, lens, ks, 16, device, seed,
                 top_k=top_k)


def config4(device, seed: int = 3, batch: int = 4, seq_len: int = 65536, steps: int = 64,
            top_k: int = 2048, page_size: int = 1) -> Workload:
    """Selection-cache trace base: tables (per token, or pages of ``page_size`` tokens)
    with free pages for ``steps`` appended tokens per request."""
    extra = batch * (-(-steps // page_size) + 1)
    return build("C4 llama3-8b B%d L%d trace page%d" % (batch, seq_len, page_size), LLAMA3_8B,
                 [seq_len] * batch, [top_k] * batch, page_size, device, seed, extra_pages=extra)


def config5_layer(device, seed: int = 4, batch: int = 4, seq_len: int = 262144,
                  top_k: int = 4096) -> Workload:
    """One layer of the full-model configuration: Llama-3-8B shape, four requests of
    256K context each, top-k 4096, page size 16."""
    return build("C5-layer llama3-8b B%d L%d k%d page16" % (batch, seq_len, top_k), LLAMA3_8B,
                 [seq_len] * batch, [top_k] * batch, 16, device, seed)


def ar1_queries(batch: int, dim: int, steps: int, device, seed: int = 3, rho: float = 0.95,
                jump_p: float = 0.1) -> torch.Tensor:
    """``q_t = rho q_{t-1} + sqrt(1-rho^2) eps`` with a fresh N(0,1) draw per
    (request, step) with probability ``jump_p``: ``[steps, batch, dim]`` bf16."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed + 1000)
    out = torch.empty((steps, batch, dim), dtype=torch.float32, device=device)
    cur = torch.randn((batch, dim), generator=gen, device=device)
    for t in range(steps):
        if t > 0:
            eps = torch.randn((batch, dim), generator=gen, device=device)
            jump = torch.rand((batch, 1), generator=gen, device=device) < jump_p
            cur = torch.where(jump, eps, rho * cur + (1 - rho * rho) ** 0.5 * eps)
        out[t] = cur
    return out.to(torch.bfloat16)
