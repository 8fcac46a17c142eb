"""Tensor-level entry points over the C ABI of ``libtokenselect_hip.so``.

PyTorch is plumbing here: it owns device memory and the HIP stream.  Every
function checks dtype / device / contiguity / shapes on the host, then passes raw
pointers and the current stream to the library.  Nothing is computed in Python
and there is no fallback path.
"""

import ctypes
import dataclasses
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import TsBatch, TsConfig, TsPagePool, TsSelCache

HEAD_DIM = 128


@dataclass
class LayerConfig:
    """The reference's module globals (tr.py:29-39) plus the attention scalars a
    ``RadixAttention`` carries (tr.py:816-822), for one layer shape."""
    num_heads: int
    num_kv_heads: int
    head_dim: int = HEAD_DIM
    page_size: int = 1
    n_init: int = 1
    n_local: int = 16
    top_k: int = 16
    pool_kernel: int = -1
    head_map: str = "mod"          # scoring: kv = h % Hkv (tr.py:202)
    rope_mode: str = "ROPE_LLAMA"  # attention: in-kernel RoPE (tr.py:822)
    rope_theta: float = 1e6
    rope_scale: float = 1.0
    sm_scale: Optional[float] = None
    logit_cap: float = 0.0

    def to_c(self) -> TsConfig:
        sm = self.sm_scale if self.sm_scale is not None else self.head_dim ** -0.5
        return TsConfig(
            self.num_heads, self.num_kv_heads, self.head_dim, self.page_size, self.n_init,
            self.n_local, self.top_k, self.pool_kernel,
            _lib.TS_HEADMAP_MOD if self.head_map == "mod" else _lib.TS_HEADMAP_DIV,
            _lib.TS_ROPE_LLAMA if self.rope_mode == "ROPE_LLAMA" else _lib.TS_ROPE_NONE,
            float(self.rope_theta), float(self.rope_scale), float(sm), float(self.logit_cap))

    @property
    def max_sel(self) -> int:
        return self.n_init + self.top_k + self.n_local


@dataclass
class Batch:
    """Running requests of a decode step.  ``table`` is ``[B, pages]`` int32
    (logical page -> physical page; with ``page_size`` 1 it is the reference's
    ``token_indices`` row, tr.py:293-297); ``seq_lens`` is ``[B]`` int32 on the
    device; ``max_seq_len`` is the host's upper bound of it."""
    seq_lens: torch.Tensor
    table: torch.Tensor
    max_seq_len: int
    k_per_req: Optional[torch.Tensor] = None
    # One int32 word of pinned host memory (see fault_word()) that the single-launch
    # selection sets to 1 when one of its grid-wide waits gave up, or None.
    fault: Optional[torch.Tensor] = None
    # Upper bounds of seq_lens that the host knows ([B] int32 on the CPU, e.g. a serving
    # framework's CPU copy of the lengths), or None: a batch too large for one selection
    # launch is then scored in phases packed by these bounds instead of by max_seq_len.
    host_seq_lens: Optional[torch.Tensor] = None
    # [B] int32 on the device, zero before a request's first step and kept per (request,
    # layer) across decode steps, or None: where the single-launch selection notes where the
    # k-th vote lay, as a guess for the next step (ts_batch.threshold_hint).
    hint: Optional[torch.Tensor] = None
    # Per-call options (``ts_batch``): take the separate kernels for this call; the call
    # repeats the step's previous one after a give-up; bound of a grid-wide wait in
    # microseconds (0: the library's 10 ms); workgroups that never arrive (tests of the
    # give-up path only).
    separate_kernels: bool = False
    rerun: bool = False
    wait_us: int = 0
    absent_workgroups: int = 0
    # ``ts_batch.workspace_clean``: the workspace was left by a completed call of the same
    # shape without a selection cache (set by :class:`DecodeLayer`, which knows).
    workspace_clean: bool = False

    @property
    def batch(self) -> int:
        return int(self.seq_lens.shape[0])


class SelectionGaveUp(RuntimeError):
    """A grid-wide wait of a fused selection kernel ran into its bound: the launch did
    not have the device to itself (its workgroups were not all resident together) and
    what it selected, and what was attended over, is not valid.  Also raised when a
    request was longer on the device than ``Batch.host_seq_lens`` said.  Raised only for
    a give-up that nobody recovered at a synchronisation point (``recover()``); the object
    that raises has switched itself to the separate kernels, so retrying works."""


def fault_word() -> torch.Tensor:
    """A zeroed int32 word of pinned host memory.  The device maps such memory, so a
    kernel can set it and the host can read it at any time without synchronising."""
    return torch.zeros((1,), dtype=torch.int32).pin_memory()


def gave_up(word: Optional[torch.Tensor]) -> bool:
    """Whether ``word`` has been set by an earlier launch.  A plain host read: a set word
    is seen at the latest after the next synchronisation."""
    return word is not None and int(word[0]) != 0


_GAVE_UP_MESSAGE = (
    "a fused selection kernel gave up waiting for its workgroups (is another stream or process "
    "using the GPU?), or a request was longer than its entry of host_seq_lens; results since the "
    "last check are not valid.  Rerun the step with the separate kernels (Batch.separate_kernels, "
    "or recover() of the layer object)")


def raise_if_gave_up(word: Optional[torch.Tensor]) -> None:
    """Raises SelectionGaveUp when ``word`` has been set by an earlier launch."""
    if gave_up(word):
        raise SelectionGaveUp(_GAVE_UP_MESSAGE)


class _GiveUpLatch:
    """What DecodeLayer and PrefillChunk share: the pinned fault word, the switch to the
    separate kernels that a give-up latches for the object, and the options of a call."""

    def _init_latch(self):
        self.fault = fault_word()
        self.separate = False  # latched by a give-up: the separate kernels from then on

    def gave_up(self) -> bool:
        """Whether a selection of this object gave up since the last check (a host memory
        read; meaningful once the stream has been synchronised)."""
        return gave_up(self.fault)

    def _latch(self) -> None:
        self.separate = True
        self.fault.zero_()

    def check(self) -> None:
        """For callers that did not recover a give-up where they synchronised: switches the
        object to the separate kernels, clears the word and raises SelectionGaveUp (the
        outputs since the last check are not valid; a retry now succeeds).  Runs at the
        start of every call."""
        if self.gave_up():
            self._latch()
            raise SelectionGaveUp(_GAVE_UP_MESSAGE + "; this object now uses the separate kernels")

    def _options(self, bt: "Batch", rerun: bool = False) -> "Batch":
        kw = {}
        if bt.fault is None:
            kw["fault"] = self.fault
        if self.separate and not bt.separate_kernels:
            kw["separate_kernels"] = True
        if rerun:
            kw["rerun"] = True
            kw["absent_workgroups"] = 0
        return dataclasses.replace(bt, **kw) if kw else bt


@dataclass
class SelectionCache:
    """Selection-cache state of one layer (tr.py:301-322)."""
    q_cache: torch.Tensor      # [B, H*D] bf16
    topk_cache: torch.Tensor   # [B, top_k] int32
    cache_len: torch.Tensor    # [B] int32
    counters: torch.Tensor     # [B, 2] int64: skip_count, retrieval_count
    threshold: float

    @classmethod
    def allocate(cls, cfg: LayerConfig, batch: int, device, threshold: Optional[float] = None):
        if threshold is None:  # 0.9 stored in bf16 (tr.py:313-315)
            threshold = float(torch.tensor(0.9, dtype=torch.bfloat16))
        return cls(
            torch.zeros((batch, cfg.num_heads * cfg.head_dim), dtype=torch.bfloat16, device=device),
            torch.zeros((batch, cfg.top_k), dtype=torch.int32, device=device),
            torch.zeros((batch,), dtype=torch.int32, device=device),
            torch.zeros((batch, 2), dtype=torch.int64, device=device), threshold)


# ------------------------------------------------------------------ helpers
def _p(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t: torch.Tensor, name: str, dtype, ndim: Optional[int] = None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device}); there is no CPU path")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if ndim is not None and t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")


def _check_pool(cfg: LayerConfig, pool: torch.Tensor, name: str):
    _need(pool, name, torch.bfloat16, 3)
    if pool.shape[1] != cfg.num_kv_heads or pool.shape[2] != cfg.head_dim:
        raise ValueError(f"{name} must be [rows, {cfg.num_kv_heads}, {cfg.head_dim}], "
                         f"got {tuple(pool.shape)}")


def _c_batch(cfg: LayerConfig, bt: Batch) -> TsBatch:
    _need(bt.seq_lens, "seq_lens", torch.int32, 1)
    _need(bt.table, "table", torch.int32, 2)
    if bt.table.shape[0] != bt.batch:
        raise ValueError("table must have one row per request")
    if bt.table.shape[1] * cfg.page_size < bt.max_seq_len:
        raise ValueError(f"table row of {bt.table.shape[1]} pages (page_size {cfg.page_size}) "
                         f"cannot address max_seq_len {bt.max_seq_len}")
    if bt.k_per_req is not None:
        _need(bt.k_per_req, "k_per_req", torch.int32, 1)
        if bt.k_per_req.shape[0] != bt.batch:
            raise ValueError("k_per_req must have one entry per request")
    if bt.fault is not None and (bt.fault.dtype != torch.int32 or bt.fault.numel() != 1 or
                                 not (bt.fault.is_cuda or bt.fault.is_pinned())):
        raise ValueError("fault must be one int32 word of device or pinned host memory")
    if bt.host_seq_lens is not None and (
            bt.host_seq_lens.dtype != torch.int32 or bt.host_seq_lens.is_cuda or
            bt.host_seq_lens.dim() != 1 or bt.host_seq_lens.shape[0] != bt.batch or
            not bt.host_seq_lens.is_contiguous()):
        raise ValueError("host_seq_lens must be a contiguous [B] int32 tensor on the CPU")
    host = bt.host_seq_lens.data_ptr() if bt.host_seq_lens is not None else None
    if bt.hint is not None:
        _need(bt.hint, "hint", torch.int32, 1)
        if bt.hint.shape[0] != bt.batch:
            raise ValueError("hint must have one entry per request")
    return TsBatch(bt.batch, int(bt.max_seq_len), _p(bt.seq_lens), _p(bt.table),
                   int(bt.table.stride(0)), _p(bt.k_per_req), _p(bt.fault), host, _p(bt.hint),
                   1 if bt.separate_kernels else 0, 1 if bt.rerun else 0, int(bt.wait_us),
                   int(bt.absent_workgroups), 1 if bt.workspace_clean else 0)


def _c_cache(cache: Optional[SelectionCache], cfg: LayerConfig, batch: int):
    if cache is None:
        return None
    _need(cache.q_cache, "q_cache", torch.bfloat16, 2)
    _need(cache.topk_cache, "topk_cache", torch.int32, 2)
    _need(cache.cache_len, "cache_len", torch.int32, 1)
    _need(cache.counters, "counters", torch.int64, 2)
    if (tuple(cache.q_cache.shape) != (batch, cfg.num_heads * cfg.head_dim)
            or tuple(cache.topk_cache.shape) != (batch, cfg.top_k)
            or cache.cache_len.shape[0] != batch or tuple(cache.counters.shape) != (batch, 2)):
        raise ValueError("selection cache arrays do not match batch / config")
    return ctypes.byref(TsSelCache(_p(cache.q_cache), _p(cache.topk_cache), _p(cache.cache_len),
                                   _p(cache.counters), float(cache.threshold)))


def set_fused_select(enable: bool) -> bool:
    """Chooses between the single-launch selection (default, where the shape allows)
    and the separate kernels inside :class:`DecodeLayer`; returns the previous
    setting."""
    return bool(_lib.load().ts_set_fused_select(1 if enable else 0))


def score_stride_for(max_seq_len: int) -> int:
    """Row stride of the score / vote buffers: ``ts_score_stride`` (a multiple of 64
    elements that keeps head rows off a power-of-two distance)."""
    return int(_lib.load().ts_score_stride(int(max_seq_len)))


# ------------------------------------------------------------- entry points
def rope_apply(x: torch.Tensor, cos_table: torch.Tensor, sin_table: torch.Tensor,
               position_ids: Optional[torch.Tensor]) -> torch.Tensor:
    """``RotaryEmbedding.apply_rotary_pos_emb`` (tr.py:98-107).  ``x`` is
    ``[rows, heads, dim]`` bf16; tables ``[T, dim]`` fp32; ``position_ids`` int64
    ``[rows]`` (``None``: every row uses table row 0)."""
    _need(x, "x", torch.bfloat16, 3)
    _need(cos_table, "cos_table", torch.float32, 2)
    _need(sin_table, "sin_table", torch.float32, 2)
    rows, heads, dim = x.shape
    if cos_table.shape != sin_table.shape or cos_table.shape[1] != dim:
        raise ValueError("cos/sin tables must both be [T, dim]")
    if position_ids is not None:
        _need(position_ids, "position_ids", torch.int64, 1)
        if position_ids.shape[0] != rows:
            raise ValueError("position_ids must have one entry per row")
    out = torch.empty_like(x)
    _lib.check(_lib.load().ts_rope_apply(_p(x), _p(out), _p(cos_table), _p(sin_table),
                                         _p(position_ids), cos_table.shape[0], rows, heads, dim,
                                         _stream()))
    return out


def paged_matmul(query: torch.Tensor, token: torch.Tensor, indices: torch.Tensor,
                 scores: torch.Tensor, num_relevant_tokens: int, num_heads: int,
                 num_kv_heads: int, head_dim: int) -> None:
    """tr.py:234-261: fills ``scores[h, t]`` (bf16 or fp32) in place."""
    _need(query, "query", torch.bfloat16)
    _need(token, "token", torch.bfloat16, 3)
    _need(indices, "indices", torch.int32, 1)
    if scores.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError("scores must be float32 or bfloat16")
    _need(scores, "scores", scores.dtype, 2)
    if query.numel() != num_heads * head_dim:
        raise ValueError("query must hold num_heads*head_dim elements")
    if token.shape[1] != num_kv_heads or token.shape[2] != head_dim:
        raise ValueError("token must be [rows, num_kv_heads, head_dim]")
    if indices.shape[0] < num_relevant_tokens or tuple(scores.shape) != (num_heads, num_relevant_tokens):
        raise ValueError("indices / scores do not match num_relevant_tokens")
    dt = _lib.TS_DTYPE_F32 if scores.dtype == torch.float32 else _lib.TS_DTYPE_BF16
    _lib.check(_lib.load().ts_paged_matmul(_p(query), _p(token), token.shape[0], _p(indices),
                                           _p(scores), dt, num_relevant_tokens, num_heads,
                                           num_kv_heads, head_dim, _stream()))


def score(cfg: LayerConfig, bt: Batch, qf: torch.Tensor, k_pool: torch.Tensor,
          skip: Optional[torch.Tensor] = None, out: Optional[Tuple] = None):
    """Scoring pass (tr.py:350-359), one kernel launch.  Returns ``(scores,
    partials)``.  ``scores`` is fp32 ``[B, stride/16, H, 16]``: tile-major, 16
    candidates per tile, head slots ``kvh*G + g`` inside a tile (see
    :func:`scores_head_major`); only the first ``L_b - n_init - n_local``
    candidates of a non-dense request are written.  ``partials`` are the
    per-workgroup softmax statistics that :func:`vote` merges."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(qf, "qf", torch.bfloat16)
    _check_pool(cfg, k_pool, "k_pool")
    B, H = bt.batch, cfg.num_heads
    if qf.numel() != B * H * cfg.head_dim:
        raise ValueError("qf must hold B*H*D elements")
    if skip is not None:
        _need(skip, "skip", torch.int32, 1)
    lib = _lib.load()
    if out is None:
        stride = score_stride_for(bt.max_seq_len)
        scores = torch.empty((B, stride // 16, H, 16), dtype=torch.float32, device=qf.device)
        nbytes = lib.ts_score_partials_bytes(ctypes.byref(c), B, bt.max_seq_len)
        partials = torch.empty((max(nbytes, 256) // 4,), dtype=torch.float32, device=qf.device)
    else:
        scores, partials = out
        _need(scores, "scores", torch.float32, 4)
        _need(partials, "partials", torch.float32, 1)
    if scores.shape[0] != B or scores.shape[2] != H or scores.shape[3] != 16:
        raise ValueError("scores must be [B, stride/16, H, 16]")
    _lib.check(lib.ts_score(ctypes.byref(c), ctypes.byref(cb), _p(qf), _p(k_pool), k_pool.shape[0],
                            _p(skip), _p(scores), scores.shape[1] * 16, _p(partials),
                            partials.numel() * 4, _stream()))
    return scores, partials


def score_buffers(cfg: LayerConfig, bt: Batch, device):
    """``(scores, partials)`` for :func:`score`'s ``out``, sized for ``bt.max_seq_len``
    (serves every shorter batch of the same size)."""
    c = cfg.to_c()
    stride = score_stride_for(bt.max_seq_len)
    scores = torch.empty((bt.batch, stride // 16, cfg.num_heads, 16), dtype=torch.float32, device=device)
    nbytes = _lib.load().ts_score_partials_bytes(ctypes.byref(c), bt.batch, bt.max_seq_len)
    partials = torch.empty((max(nbytes, 256) // 4,), dtype=torch.float32, device=device)
    return scores, partials


def select_supported(cfg: LayerConfig, batch: int, max_seq_len: int) -> bool:
    """Whether :func:`select` can serve this shape (``ts_select_supported``)."""
    return bool(_lib.load().ts_select_supported(ctypes.byref(cfg.to_c()), int(batch),
                                                int(max_seq_len)))


def select_clear(cfg: LayerConfig, bt: Batch, workspace: torch.Tensor) -> None:
    """Clears what :func:`select` with ``cleared=True`` wants zero in ``workspace``."""
    _lib.check(_lib.load().ts_select_clear(ctypes.byref(cfg.to_c()), ctypes.byref(_c_batch(cfg, bt)),
                                           _p(workspace), workspace.numel(), _stream()))


def select_workspace(cfg: LayerConfig, bt: Batch, device) -> torch.Tensor:
    nbytes = _lib.load().ts_select_workspace_bytes(ctypes.byref(cfg.to_c()), bt.batch, bt.max_seq_len)
    return torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=device)


def select(cfg: LayerConfig, bt: Batch, qf: torch.Tensor, k_pool: torch.Tensor,
           hit: Optional[torch.Tensor] = None, cache: Optional[SelectionCache] = None,
           want_votes: bool = False, workspace: Optional[torch.Tensor] = None,
           cleared: bool = False, wait_ticks: Optional[int] = None, absent_workgroups: int = 0):
    """The whole selection in one launch (tr.py:350-373, 424-449): scoring, soft vote,
    exact top-k, ascending order and index assembly, the scores never leaving LDS.
    Returns ``(sel, sel_pos, sel_len, votes, workspace)`` with the first three as
    from :func:`topk_ragged`; ``votes`` is ``[B, stride]`` fp32 when ``want_votes``
    else ``None``.  ``workspace`` (uint8) may be passed back in to avoid allocating;
    with ``cleared`` the caller has run :func:`select_clear` on it since its last use
    and only the selection kernel is launched.  ``wait_ticks`` / ``absent_workgroups``
    go to ``ts_select_cleared_bounded`` (tests of the give-up path).  A launch that gave
    up reports ``sel_len[b] == -1`` and sets ``bt.fault``."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(qf, "qf", torch.bfloat16)
    _check_pool(cfg, k_pool, "k_pool")
    B = bt.batch
    if qf.numel() != B * cfg.num_heads * cfg.head_dim:
        raise ValueError("qf must hold B*H*D elements")
    if hit is not None:
        _need(hit, "hit", torch.int32, 1)
    lib = _lib.load()
    nbytes = lib.ts_select_workspace_bytes(ctypes.byref(c), B, bt.max_seq_len)
    if cleared and (workspace is None or workspace.numel() < nbytes):
        raise ValueError("cleared=True needs the workspace that select_clear was run on")
    if workspace is None or workspace.numel() < nbytes:
        workspace = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=qf.device)
    sel = torch.empty((B, cfg.max_sel), dtype=torch.int32, device=qf.device)
    sel_pos = torch.empty_like(sel)
    sel_len = torch.empty((B,), dtype=torch.int32, device=qf.device)
    votes = None
    if want_votes:
        votes = torch.empty((B, score_stride_for(bt.max_seq_len)), dtype=torch.float32,
                            device=qf.device)
    args = (ctypes.byref(c), ctypes.byref(cb), _p(qf), _p(k_pool), k_pool.shape[0], _p(hit),
            _c_cache(cache, cfg, B), _p(sel), _p(sel_pos), cfg.max_sel, _p(sel_len), _p(votes),
            votes.shape[1] if votes is not None else 0, _p(workspace), workspace.numel())
    if wait_ticks is not None or absent_workgroups:
        if not cleared:
            _lib.check(lib.ts_select_clear(ctypes.byref(c), ctypes.byref(cb), _p(workspace),
                                           workspace.numel(), _stream()))
        _lib.check(lib.ts_select_cleared_bounded(
            *args, int(wait_ticks if wait_ticks is not None else 200_000_000),
            int(absent_workgroups), _stream()))
    else:
        _lib.check((lib.ts_select_cleared if cleared else lib.ts_select)(*args, _stream()))
    return sel, sel_pos, sel_len, votes, workspace


def select_fault(cfg: LayerConfig, bt: Batch, workspace: torch.Tensor) -> bool:
    """True when a grid-wide wait of the last :func:`select` on ``workspace`` gave up
    (synchronises)."""
    nbytes = _lib.load().ts_select_workspace_bytes(ctypes.byref(cfg.to_c()), bt.batch,
                                                   bt.max_seq_len)
    # the rendezvous areas (one of 65 x 4096 bytes per request) end the workspace; the
    # fault word is the first word of the first
    return bool(workspace.view(torch.int32)[nbytes // 4 - bt.batch * 65 * 1024].item())


def select_rounds(cfg: LayerConfig, bt: Batch, workspace: torch.Tensor, rounds: int = 4):
    """How many groups of workgroups completed each grid-wide round of the last
    :func:`select` on ``workspace`` (synchronises): a round nobody met for shows zero."""
    nbytes = _lib.load().ts_select_workspace_bytes(ctypes.byref(cfg.to_c()), bt.batch,
                                                   bt.max_seq_len)
    first = nbytes // 4 - bt.batch * 65 * 1024
    return workspace.view(torch.int32)[first + 2:first + 2 + rounds].tolist()


def scores_head_major(cfg: LayerConfig, scores: torch.Tensor) -> torch.Tensor:
    """``[B, H, stride]`` view-copy of the tile-major scores, rows in true head
    order (slot ``kvh*G + g`` is head ``kvh + Hkv*g`` under the reference's ``%``
    map, head ``kvh*G + g`` under the conventional one)."""
    B, tiles, H, _ = scores.shape
    group = H // cfg.num_kv_heads
    slots = torch.arange(H, device=scores.device)
    heads = (slots // group) + cfg.num_kv_heads * (slots % group) if cfg.head_map == "mod" else slots
    out = torch.empty((B, H, tiles * 16), dtype=scores.dtype, device=scores.device)
    out[:, heads] = scores.permute(0, 2, 1, 3).reshape(B, H, tiles * 16)
    return out


def vote(cfg: LayerConfig, bt: Batch, scores: torch.Tensor, partials: torch.Tensor,
         skip: Optional[torch.Tensor] = None):
    """Soft vote (tr.py:361) and optional max-pool (tr.py:366-369).  Returns
    ``(votes [B, stride] fp32, stats [B,H,2] fp32 = per-head (max, sum exp))``."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(scores, "scores", torch.float32, 4)
    _need(partials, "partials", torch.float32, 1)
    B, H = bt.batch, cfg.num_heads
    if scores.shape[0] != B or scores.shape[2] != H or scores.shape[3] != 16:
        raise ValueError("scores must be [B, stride/16, H, 16]")
    lib = _lib.load()
    if partials.numel() * 4 < lib.ts_score_partials_bytes(ctypes.byref(c), B, bt.max_seq_len):
        raise ValueError("partials buffer is smaller than ts_score_partials_bytes()")
    stride = scores.shape[1] * 16
    stats = torch.empty((B, H, 2), dtype=torch.float32, device=scores.device)
    votes = torch.empty((B, stride), dtype=torch.float32, device=scores.device)
    pooled = torch.empty_like(votes) if cfg.pool_kernel > 0 else None
    _lib.check(lib.ts_vote(ctypes.byref(c), ctypes.byref(cb), _p(scores), stride, _p(partials),
                           _p(skip), _p(stats), _p(votes), _p(pooled), stride, _stream()))
    return (pooled if pooled is not None else votes), stats


def layer_selection_form(cfg: LayerConfig, batch, max_seq_len: Optional[int] = None) -> int:
    """How :class:`DecodeLayer` selects for a shape ``(batch, max_seq_len)`` or for a
    :class:`Batch`: 2 = one ``ts_select`` launch, 1 = ``ts_score_vote``'s launch + the top-k
    kernels, 0 = the separate kernels."""
    if isinstance(batch, Batch):
        cb = _c_batch(cfg, batch)
        return int(_lib.load().ts_decode_layer_selection_of(ctypes.byref(cfg.to_c()), ctypes.byref(cb)))
    return int(_lib.load().ts_decode_layer_selection(ctypes.byref(cfg.to_c()), int(batch),
                                                     int(max_seq_len)))


def score_vote_supported(cfg: LayerConfig, batch: int, max_seq_len: int) -> bool:
    """Whether :func:`score_vote` can serve this shape (``ts_score_vote_supported``)."""
    return bool(_lib.load().ts_score_vote_supported(ctypes.byref(cfg.to_c()), int(batch),
                                                    int(max_seq_len)))


def score_vote(cfg: LayerConfig, bt: Batch, qf: torch.Tensor, k_pool: torch.Tensor,
               skip: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None):
    """:func:`score` + :func:`vote` without the scores in memory (``ts_score_vote``), a
    batch of any size, its requests in phases that fit the LDS of the device.  Returns
    ``votes [B, stride]`` fp32 (pooled when ``cfg.pool_kernel > 0``)."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(qf, "qf", torch.bfloat16)
    _check_pool(cfg, k_pool, "k_pool")
    B = bt.batch
    if qf.numel() != B * cfg.num_heads * cfg.head_dim:
        raise ValueError("qf must hold B*H*D elements")
    if skip is not None:
        _need(skip, "skip", torch.int32, 1)
    lib = _lib.load()
    nbytes = lib.ts_select_workspace_bytes(ctypes.byref(c), B, bt.max_seq_len)
    if workspace is None or workspace.numel() < nbytes:
        workspace = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=qf.device)
    votes = torch.empty((B, score_stride_for(bt.max_seq_len)), dtype=torch.float32, device=qf.device)
    _lib.check(lib.ts_score_vote(ctypes.byref(c), ctypes.byref(cb), _p(qf), _p(k_pool), k_pool.shape[0],
                                 _p(skip), _p(votes), votes.shape[1], _p(workspace), workspace.numel(),
                                 _stream()))
    return votes


def topk_ragged(cfg: LayerConfig, bt: Batch, votes: torch.Tensor,
                hit: Optional[torch.Tensor] = None, cache: Optional[SelectionCache] = None):
    """Top-k + sort + assembly (tr.py:371-373, 433-449).  Returns
    ``(sel [B,max_sel] int32 physical slots, sel_pos [B,max_sel] int32 logical
    positions, sel_len [B] int32)``."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(votes, "votes", torch.float32, 2)
    B = bt.batch
    if votes.shape[0] != B:
        raise ValueError("votes must have one row per request")
    if hit is not None:
        _need(hit, "hit", torch.int32, 1)
    sel = torch.empty((B, cfg.max_sel), dtype=torch.int32, device=votes.device)
    sel_pos = torch.empty_like(sel)
    sel_len = torch.empty((B,), dtype=torch.int32, device=votes.device)
    lib = _lib.load()
    nbytes = lib.ts_topk_workspace_bytes(ctypes.byref(c), B, bt.max_seq_len)
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=votes.device)
    _lib.check(lib.ts_topk_ragged(ctypes.byref(c), ctypes.byref(cb), _p(votes), votes.shape[1], _p(hit),
                     _c_cache(cache, cfg, B), _p(sel), _p(sel_pos), cfg.max_sel, _p(sel_len), _p(ws),
                     ws.numel(), _stream()))
    return sel, sel_pos, sel_len


def selcache_step(cfg: LayerConfig, bt: Batch, qf: torch.Tensor, cache: SelectionCache) -> torch.Tensor:
    """Selection-cache decision (tr.py:394-401, 416-421): ``hit [B]`` int32."""
    c, cb = cfg.to_c(), _c_batch(cfg, bt)
    _need(qf, "qf", torch.bfloat16)
    if qf.numel() != bt.batch * cfg.num_heads * cfg.head_dim:
        raise ValueError("qf must hold B*H*D elements")
    hit = torch.empty((bt.batch,), dtype=torch.int32, device=qf.device)
    _lib.check(_lib.load().ts_selcache_step(ctypes.byref(c), ctypes.byref(cb), _p(qf),
                                            _c_cache(cache, cfg, bt.batch), _p(hit), _stream()))
    return hit


def sparse_decode_attention(cfg: LayerConfig, q: torch.Tensor, k_pool: torch.Tensor,
                            v_pool: torch.Tensor, sel: torch.Tensor, sel_len: torch.Tensor,
                            max_sel_len: Optional[int] = None) -> torch.Tensor:
    """Decode attention over the selected slots (tr.py:815-823): ``[B, H*D]`` bf16."""
    c = cfg.to_c()
    _need(q, "q", torch.bfloat16)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(sel, "sel", torch.int32, 2)
    _need(sel_len, "sel_len", torch.int32, 1)
    B = sel.shape[0]
    if k_pool.shape != v_pool.shape:
        raise ValueError("k_pool and v_pool must have the same shape")
    if q.numel() != B * cfg.num_heads * cfg.head_dim or sel_len.shape[0] != B:
        raise ValueError("q / sel_len do not match the batch of sel")
    max_sel_len = sel.shape[1] if max_sel_len is None else int(max_sel_len)
    if max_sel_len > sel.shape[1]:
        raise ValueError("max_sel_len exceeds the width of sel")
    lib = _lib.load()
    out = torch.empty((B, cfg.num_heads * cfg.head_dim), dtype=torch.bfloat16, device=q.device)
    ws_bytes = lib.ts_attn_workspace_bytes(ctypes.byref(c), B, max_sel_len)
    ws = torch.empty((max(ws_bytes, 256),), dtype=torch.uint8, device=q.device)
    _lib.check(lib.ts_sparse_decode_attn(ctypes.byref(c), _p(q), _p(k_pool), _p(v_pool),
                                         k_pool.shape[0], _p(sel), sel.stride(0), _p(sel_len), B,
                                         max_sel_len, _p(out), _p(ws), ws.numel(), _stream()))
    return out


@dataclass
class PagePool:
    """Free pages of a paged KV pool (``ts_page_pool``): a stack of physical page
    numbers on the device, ``free_pages[:free_count]`` being free and the top taken
    first, plus the ticket word the store kernels count their workgroups in."""
    free_pages: torch.Tensor   # [capacity] int32
    free_count: torch.Tensor   # [1] int32
    ticket: torch.Tensor       # [1] int32, zero between calls

    @classmethod
    def of(cls, pages: torch.Tensor):
        """A pool whose free pages are ``pages`` (int32, on the device; the last one is
        taken first)."""
        _need(pages, "pages", torch.int32, 1)
        return cls(pages.clone(), torch.tensor([pages.shape[0]], dtype=torch.int32, device=pages.device),
                   torch.zeros((1,), dtype=torch.int32, device=pages.device))

    def to_c(self) -> TsPagePool:
        _need(self.free_pages, "free_pages", torch.int32, 1)
        _need(self.free_count, "free_count", torch.int32, 1)
        _need(self.ticket, "ticket", torch.int32, 1)
        return TsPagePool(_p(self.free_pages), _p(self.free_count), _p(self.ticket))


def _c_pages(cfg: LayerConfig, out_cache_loc, pages: Optional[PagePool]):
    """(out_cache_loc pointer, ts_page_pool*) for the store entry points: the caller's
    slots with a per-token table (the reference), or slots the library takes from the
    table / the page pool."""
    if pages is not None:
        c_pool = pages.to_c()
        return None, ctypes.byref(c_pool), c_pool
    if cfg.page_size != 1:
        raise ValueError(f"page_size {cfg.page_size} needs a PagePool")
    _need(out_cache_loc, "out_cache_loc", torch.int32, 1)
    return _p(out_cache_loc), None, None


def kv_store(cfg: LayerConfig, k: torch.Tensor, v: torch.Tensor, out_cache_loc: Optional[torch.Tensor],
             k_pool: torch.Tensor, v_pool: torch.Tensor, table: torch.Tensor,
             seq_lens: torch.Tensor, pages: Optional[PagePool] = None) -> None:
    """KV store + table append of a decode step (tr.py:844-854, 332-336): to the
    caller's ``out_cache_loc`` (page size 1, the reference), or, with ``pages``, to the
    next position of each request's paged table, fresh pages coming from the pool."""
    c = cfg.to_c()
    _need(k, "k", torch.bfloat16)
    _need(v, "v", torch.bfloat16)
    loc, pool, _keep = _c_pages(cfg, out_cache_loc, pages)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(table, "table", torch.int32, 2)
    _need(seq_lens, "seq_lens", torch.int32, 1)
    B = seq_lens.shape[0]
    row = cfg.num_kv_heads * cfg.head_dim
    if k.numel() != B * row or v.numel() != B * row or table.shape[0] != B or \
            (pages is None and out_cache_loc.shape[0] != B):
        raise ValueError("k / v / out_cache_loc / table / seq_lens do not match the batch")
    _lib.check(_lib.load().ts_kv_store(ctypes.byref(c), _p(k), _p(v), loc, pool, _p(k_pool),
                                       _p(v_pool), k_pool.shape[0], _p(table), table.stride(0),
                                       _p(seq_lens), B, table.shape[1] * cfg.page_size, _stream()))


QKV_STORE_MAX_BATCH = 8


def qkv_store_supported(batch: int, hidden: int) -> bool:
    """Shapes :func:`qkv_store` serves; others take a library GEMM and :func:`kv_store`."""
    return 1 <= batch <= QKV_STORE_MAX_BATCH and 8 <= hidden <= 4096 and hidden % 8 == 0


def qkv_store(cfg: LayerConfig, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
              out_cache_loc: Optional[torch.Tensor], k_pool: torch.Tensor, v_pool: torch.Tensor,
              table: torch.Tensor, seq_lens: torch.Tensor,
              q_out: Optional[torch.Tensor] = None, pages: Optional[PagePool] = None) -> torch.Tensor:
    """QKV projection of a decode step with the KV store + table append as its epilogue
    (the model's ``qkv_proj`` followed by tr.py:844-854, 332-336) in one pass over the
    weight.  ``x`` [B, hidden] bf16, ``weight`` [(H+2Hkv)*D, hidden] bf16 (a torch
    ``Linear`` weight), ``bias`` [(H+2Hkv)*D] bf16 or None.  Returns ``q`` [B, H*D] bf16;
    K and V land in the pools at ``out_cache_loc`` or, with ``pages``, where
    :func:`kv_store` would put them."""
    c = cfg.to_c()
    _need(x, "x", torch.bfloat16, 2)
    _need(weight, "weight", torch.bfloat16, 2)
    if bias is not None:
        _need(bias, "bias", torch.bfloat16, 1)
    loc, pool, _keep = _c_pages(cfg, out_cache_loc, pages)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(table, "table", torch.int32, 2)
    _need(seq_lens, "seq_lens", torch.int32, 1)
    B, hidden = x.shape
    n_out = (cfg.num_heads + 2 * cfg.num_kv_heads) * cfg.head_dim
    if tuple(weight.shape) != (n_out, hidden) or (bias is not None and bias.shape[0] != n_out):
        raise ValueError(f"weight must be [{n_out}, {hidden}] (and bias [{n_out}])")
    if (pages is None and out_cache_loc.shape[0] != B) or table.shape[0] != B or seq_lens.shape[0] != B:
        raise ValueError("out_cache_loc / table / seq_lens do not match the batch")
    if k_pool.shape != v_pool.shape:
        raise ValueError("k_pool and v_pool must have the same shape")
    if q_out is None:
        q_out = torch.empty((B, cfg.num_heads * cfg.head_dim), dtype=torch.bfloat16, device=x.device)
    else:
        _need(q_out, "q_out", torch.bfloat16, 2)
        if tuple(q_out.shape) != (B, cfg.num_heads * cfg.head_dim):
            raise ValueError("q_out must be [B, H*D]")
    _lib.check(_lib.load().ts_qkv_store(
        ctypes.byref(c), _p(x), _p(weight), _p(bias), hidden, loc, pool, _p(q_out), _p(k_pool),
        _p(v_pool), k_pool.shape[0], _p(table), table.stride(0), _p(seq_lens), B,
        table.shape[1] * cfg.page_size, _stream()))
    return q_out


def scoring_cos_sin(head_dim: int, rope_base: float, rope_scale, n_local: int, device):
    """Row ``n_local`` of the reference's cos/sin tables (tr.py:75-96), built with
    the same fp32 torch expressions on the host: ``(cos [1,D], sin [1,D])``."""
    inv_freq = 1.0 / (rope_base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    t = torch.arange(n_local + 1)
    freqs = torch.outer(t * rope_scale, inv_freq)[n_local:n_local + 1]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(device).contiguous(), emb.sin().to(device).contiguous()


class DecodeLayer(_GiveUpLatch):
    """One layer of the patched decode forward after the KV store
    (tr.py:791-825) as a single library call; buffers are allocated once.

    A fused selection kernel that gave up (``SelectionGaveUp``) has left ``sel_len[b] = -1``
    and an output attended over nothing.  A caller that synchronises before the output is
    consumed calls :meth:`recover` there with the arguments of the call: it repeats the
    step's selection and attention with the separate kernels (the KV store before the
    layer is not repeated) and keeps the object on them."""

    def __init__(self, cfg: LayerConfig, batch: int, max_seq_len: int, device):
        self.cfg, self.batch, self.max_seq_len = cfg, batch, max_seq_len
        self._c = cfg.to_c()
        lib = _lib.load()
        _lib.check(lib.ts_check_config(ctypes.byref(self._c)))
        nbytes = lib.ts_decode_layer_workspace_bytes(ctypes.byref(self._c), batch, max_seq_len)
        self.workspace = torch.empty((nbytes,), dtype=torch.uint8, device=device)
        self.q_cos, self.q_sin = scoring_cos_sin(cfg.head_dim, cfg.rope_theta, cfg.rope_scale,
                                                 cfg.n_local, device)
        self.out = torch.empty((batch, cfg.num_heads * cfg.head_dim), dtype=torch.bfloat16,
                               device=device)
        self.sel = torch.empty((batch, cfg.max_sel), dtype=torch.int32, device=device)
        self.sel_pos = torch.empty_like(self.sel)
        self.sel_len = torch.empty((batch,), dtype=torch.int32, device=device)
        self._init_latch()
        # (batch, max_seq_len) of the last call when it was a plain layer call without a
        # selection cache that raised nothing: that call's attention kernel has left the
        # selection's counters zero, and the next call of the same shape says so
        # (``ts_batch.workspace_clean``) and starts with the selection kernel.
        self._clean_for = None

    def recover(self, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch,
                cache: Optional[SelectionCache] = None, out: Optional[torch.Tensor] = None):
        """Synchronises the stream; when the last call gave up, repeats it (same
        arguments) with the separate kernels, which stay switched on for this object, and
        returns what the call returns; ``None`` when there was nothing to recover.  With
        the selection cache the requests that gave up select afresh, the others hit
        again, and the counters do not advance twice."""
        torch.cuda.current_stream().synchronize()
        if not self.gave_up():
            return None
        self._latch()
        return self._run(q, k_pool, v_pool, bt, cache, out, rerun=True)

    def __call__(self, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch,
                 cache: Optional[SelectionCache] = None, out: Optional[torch.Tensor] = None):
        self.check()
        return self._run(q, k_pool, v_pool, bt, cache, out)

    def step(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out_cache_loc: Optional[torch.Tensor],
             k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch, cache: Optional[SelectionCache] = None,
             out: Optional[torch.Tensor] = None, pages: Optional["PagePool"] = None):
        """The reference's decode forward of a layer in one call (tr.py:777-825,
        ``ts_decode_step``): :func:`kv_store` of the new token's ``k`` / ``v`` into the pools
        and ``bt.table`` / ``bt.seq_lens`` (both written), then the layer on the lengths after
        the append, which ``bt.max_seq_len`` and ``bt.host_seq_lens`` must bound.  Same
        results as the two calls; with a selection cache the store rides in the layer's
        first launch."""
        self.check()
        cfg = self.cfg
        _need(k, "k", torch.bfloat16)
        _need(v, "v", torch.bfloat16)
        loc, pool, _keep = _c_pages(cfg, out_cache_loc, pages)
        _need(bt.table, "table", torch.int32, 2)
        B = bt.batch
        row = cfg.num_kv_heads * cfg.head_dim
        if k.numel() != B * row or v.numel() != B * row or bt.table.shape[0] != B or \
                (pages is None and out_cache_loc.shape[0] != B):
            raise ValueError("k / v / out_cache_loc / table do not match the batch")
        kv = _lib.TsNewKv(_p(k), _p(v), loc, ctypes.pointer(_keep) if pages is not None else None,
                          bt.table.shape[1] * cfg.page_size)
        kv._pool = _keep  # (the struct the pointer refers to lives as long as kv)
        return self._run(q, k_pool, v_pool, bt, cache, out, new_kv=kv)

    def _run(self, q, k_pool, v_pool, bt, cache, out, rerun: bool = False, new_kv=None):
        cfg = self.cfg
        bt = self._options(bt, rerun)
        shape = (bt.batch, int(bt.max_seq_len))
        plain = cache is None and not bt.separate_kernels and not rerun
        if plain and self._clean_for == shape and not bt.workspace_clean:
            bt = dataclasses.replace(bt, workspace_clean=True)
        self._clean_for = None
        cb = _c_batch(cfg, bt)
        if bt.batch > self.batch or bt.max_seq_len > self.max_seq_len:
            raise ValueError("batch / max_seq_len exceed what this DecodeLayer was sized for")
        _need(q, "q", torch.bfloat16)
        B = bt.batch
        if q.numel() != B * cfg.num_heads * cfg.head_dim:
            raise ValueError("q must hold B*H*D elements")
        _check_pool(cfg, k_pool, "k_pool")
        _check_pool(cfg, v_pool, "v_pool")
        if k_pool.shape != v_pool.shape:
            raise ValueError("k_pool and v_pool must have the same shape")
        if out is None:
            out = self.out[:B]
        else:
            _need(out, "out", torch.bfloat16)
            if out.numel() != q.numel():
                raise ValueError("out must hold B*H*D elements")
        if new_kv is not None:
            _lib.check(_lib.load().ts_decode_step(
                ctypes.byref(self._c), ctypes.byref(cb), ctypes.byref(new_kv), _p(q), _p(self.q_cos),
                _p(self.q_sin), _p(k_pool), _p(v_pool), k_pool.shape[0], _c_cache(cache, cfg, B), _p(out),
                _p(self.sel), _p(self.sel_pos), cfg.max_sel, _p(self.sel_len), _p(self.workspace),
                self.workspace.numel(), _stream()))
        else:
            _lib.check(_lib.load().ts_decode_layer(
                ctypes.byref(self._c), ctypes.byref(cb), _p(q), _p(self.q_cos), _p(self.q_sin),
                _p(k_pool), _p(v_pool), k_pool.shape[0], _c_cache(cache, cfg, B), _p(out),
                _p(self.sel), _p(self.sel_pos), cfg.max_sel, _p(self.sel_len), _p(self.workspace),
                self.workspace.numel(), _stream()))
        if plain:
            self._clean_for = shape
        return out, self.sel[:B], self.sel_pos[:B], self.sel_len[:B]

    # The layer split at the vote (tensor parallelism, tr.py:361-364): votes() leaves this
    # rank's partial votes, the caller adds the ranks' votes in place (all-reduce), attend()
    # selects from the sum and attends with this rank's heads.
    def votes(self, q: torch.Tensor, k_pool: torch.Tensor, bt: Batch,
              cache: Optional[SelectionCache] = None) -> torch.Tensor:
        cfg = self.cfg
        self.check()
        self._clean_for = None  # (other kernels use the workspace from here on)
        bt = self._options(bt)
        cb = _c_batch(cfg, bt)
        if bt.batch > self.batch or bt.max_seq_len > self.max_seq_len:
            raise ValueError("batch / max_seq_len exceed what this DecodeLayer was sized for")
        _need(q, "q", torch.bfloat16)
        _check_pool(cfg, k_pool, "k_pool")
        B = bt.batch
        if q.numel() != B * cfg.num_heads * cfg.head_dim:
            raise ValueError("q must hold B*H*D elements")
        if getattr(self, "_votes", None) is None:
            self._votes = torch.zeros((self.batch, score_stride_for(self.max_seq_len)),
                                      dtype=torch.float32, device=q.device)
        _lib.check(_lib.load().ts_decode_layer_votes(
            ctypes.byref(self._c), ctypes.byref(cb), _p(q), _p(self.q_cos), _p(self.q_sin), _p(k_pool),
            k_pool.shape[0], _c_cache(cache, cfg, B), _p(self._votes), self._votes.shape[1],
            _p(self.workspace), self.workspace.numel(), _stream()))
        return self._votes[:B]

    def attend(self, q: torch.Tensor, votes: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
               bt: Batch, cache: Optional[SelectionCache] = None, out: Optional[torch.Tensor] = None):
        cfg = self.cfg
        self._clean_for = None
        bt = self._options(bt)
        cb = _c_batch(cfg, bt)
        _need(q, "q", torch.bfloat16)
        _need(votes, "votes", torch.float32, 2)
        _check_pool(cfg, k_pool, "k_pool")
        _check_pool(cfg, v_pool, "v_pool")
        B = bt.batch
        if q.numel() != B * cfg.num_heads * cfg.head_dim or votes.shape[0] != B:
            raise ValueError("q / votes do not match the batch")
        if out is None:
            out = self.out[:B]
        _lib.check(_lib.load().ts_decode_layer_attend(
            ctypes.byref(self._c), ctypes.byref(cb), _p(q), _p(votes), votes.stride(0), _p(k_pool),
            _p(v_pool), k_pool.shape[0], _c_cache(cache, cfg, B), _p(out), _p(self.sel),
            _p(self.sel_pos), cfg.max_sel, _p(self.sel_len), _p(self.workspace),
            self.workspace.numel(), _stream()))
        return out, self.sel[:B], self.sel_pos[:B], self.sel_len[:B]


# ---------------------------------------------------------------- chunked prefill
def rope_tables(head_dim: int, rope_base: float, rope_scale, rows: int, device):
    """The reference's cos/sin tables (tr.py:75-96) for positions ``0..rows-1``, built
    with the same fp32 torch expressions on the host: ``(cos [rows,D], sin [rows,D])``."""
    inv_freq = 1.0 / (rope_base ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(rows) * rope_scale, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(device).contiguous(), emb.sin().to(device).contiguous()


def kv_store_chunk(cfg: LayerConfig, k: torch.Tensor, v: torch.Tensor,
                   out_cache_loc: Optional[torch.Tensor], k_pool: torch.Tensor, v_pool: torch.Tensor,
                   table_row: torch.Tensor, seq_len: torch.Tensor,
                   pages: Optional[PagePool] = None) -> None:
    """KV store + table append of a prefill chunk of one request (tr.py:725-733,
    332-336): ``table_row`` [pages of the request] int32, ``seq_len`` a one-element int32
    tensor; slots from ``out_cache_loc`` (page size 1) or, with ``pages``, from the table
    and the page pool."""
    c = cfg.to_c()
    _need(k, "k", torch.bfloat16)
    _need(v, "v", torch.bfloat16)
    loc, pool, _keep = _c_pages(cfg, out_cache_loc, pages)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(table_row, "table_row", torch.int32, 1)
    _need(seq_len, "seq_len", torch.int32)
    row = cfg.num_kv_heads * cfg.head_dim
    rows = k.numel() // row
    if k.numel() != rows * row or v.numel() != rows * row or seq_len.numel() != 1 or \
            (pages is None and out_cache_loc.shape[0] != rows):
        raise ValueError("k / v / out_cache_loc / seq_len do not match the chunk")
    _lib.check(_lib.load().ts_kv_store_chunk(ctypes.byref(c), _p(k), _p(v), loc, pool, rows,
                                             _p(k_pool), _p(v_pool), k_pool.shape[0], _p(table_row),
                                             _p(seq_len), table_row.shape[0] * cfg.page_size,
                                             _stream()))


def fingerprint(cfg: LayerConfig, q: torch.Tensor, cos_table: torch.Tensor,
                sin_table: torch.Tensor) -> torch.Tensor:
    """Fingerprint of a chunk (tr.py:380-392): ``q`` [rows, H, D] bf16, row ``i``
    rotated to ``n_local + i``, mean over the rows: ``[H, D]`` bf16."""
    _need(q, "q", torch.bfloat16, 3)
    _need(cos_table, "cos_table", torch.float32, 2)
    _need(sin_table, "sin_table", torch.float32, 2)
    rows, H, D = q.shape
    if H != cfg.num_heads or D != cfg.head_dim or cos_table.shape != sin_table.shape \
            or cos_table.shape[1] != D:
        raise ValueError("q must be [rows, H, D] and the tables [T, D]")
    qf = torch.empty((H, D), dtype=torch.bfloat16, device=q.device)
    _lib.check(_lib.load().ts_fingerprint(ctypes.byref(cfg.to_c()), _p(q), rows, _p(cos_table),
                                          _p(sin_table), cos_table.shape[0], _p(qf), _stream()))
    return qf


def sparse_prefill_attention(cfg: LayerConfig, q: torch.Tensor, k_pool: torch.Tensor,
                             v_pool: torch.Tensor, sel: torch.Tensor, sel_len: torch.Tensor,
                             max_sel_len: Optional[int] = None) -> torch.Tensor:
    """Causal attention of a chunk over the selected slots (tr.py:759-771): ``q``
    [rows, H*D] bf16, ``sel`` [>= max_sel_len] int32, ``sel_len`` one-element int32."""
    _need(q, "q", torch.bfloat16, 2)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(sel, "sel", torch.int32)
    _need(sel_len, "sel_len", torch.int32)
    rows = q.shape[0]
    if q.shape[1] != cfg.num_heads * cfg.head_dim:
        raise ValueError("q must be [rows, H*D]")
    if max_sel_len is None:
        max_sel_len = sel.numel()
    if sel.numel() < max_sel_len or sel_len.numel() != 1:
        raise ValueError("sel shorter than max_sel_len, or sel_len not a scalar")
    out = torch.empty_like(q)
    lib, c = _lib.load(), cfg.to_c()
    nbytes = lib.ts_prefill_attn_workspace_bytes(ctypes.byref(c), max_sel_len)
    ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=q.device)
    _lib.check(lib.ts_sparse_prefill_attn(ctypes.byref(c), _p(q), rows, _p(k_pool), _p(v_pool),
                                          k_pool.shape[0], _p(sel), _p(sel_len), max_sel_len, _p(out),
                                          _p(ws), ws.numel(), _stream()))
    return out


class PrefillChunk(_GiveUpLatch):
    """One chunk of the patched extend forward after its KV store (tr.py:735-773) as a
    single library call, for one request; buffers are allocated once.  :meth:`recover`
    as for :class:`DecodeLayer`."""

    def __init__(self, cfg: LayerConfig, max_seq_len: int, device, max_rows: int = 512):
        self.cfg, self.max_seq_len, self.max_rows = cfg, max_seq_len, max_rows
        self._c = cfg.to_c()
        lib = _lib.load()
        _lib.check(lib.ts_check_config(ctypes.byref(self._c)))
        nbytes = lib.ts_decode_layer_workspace_bytes(ctypes.byref(self._c), 1, max_seq_len)
        self.workspace = torch.empty((nbytes,), dtype=torch.uint8, device=device)
        self.cos, self.sin = rope_tables(cfg.head_dim, cfg.rope_theta, cfg.rope_scale,
                                         cfg.n_local + max_rows, device)
        self.sel = torch.empty((1, cfg.max_sel), dtype=torch.int32, device=device)
        self.sel_pos = torch.empty_like(self.sel)
        self.sel_len = torch.empty((1,), dtype=torch.int32, device=device)
        self._init_latch()

    def recover(self, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch,
                out: Optional[torch.Tensor] = None):
        """As :meth:`DecodeLayer.recover`: after a synchronisation, repeats a chunk whose
        selection gave up with the separate kernels; ``None`` when nothing gave up."""
        torch.cuda.current_stream().synchronize()
        if not self.gave_up():
            return None
        self._latch()
        return self._run(q, k_pool, v_pool, bt, out, rerun=True)

    def __call__(self, q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch,
                 out: Optional[torch.Tensor] = None):
        self.check()
        return self._run(q, k_pool, v_pool, bt, out)

    def step(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out_cache_loc: Optional[torch.Tensor],
             k_pool: torch.Tensor, v_pool: torch.Tensor, bt: Batch, out: Optional[torch.Tensor] = None,
             pages: Optional["PagePool"] = None):
        """One chunk of the extend forward in one call (tr.py:725-773, ``ts_prefill_step``):
        :func:`kv_store_chunk` of the chunk's ``k`` / ``v`` into the pools and ``bt.table`` /
        ``bt.seq_lens`` (both written), then the chunk on the length after the append, which
        ``bt.max_seq_len`` must bound.  Same results as the two calls; with caller-chosen
        slots the store rides in the chunk's first launch."""
        self.check()
        cfg = self.cfg
        _need(k, "k", torch.bfloat16)
        _need(v, "v", torch.bfloat16)
        loc, pool, _keep = _c_pages(cfg, out_cache_loc, pages)
        _need(bt.table, "table", torch.int32, 2)
        row = cfg.num_kv_heads * cfg.head_dim
        rows = q.shape[0]
        if k.numel() != rows * row or v.numel() != rows * row or bt.table.shape[0] != 1 or \
                (pages is None and out_cache_loc.shape[0] != rows):
            raise ValueError("k / v / out_cache_loc / table do not match the chunk")
        kv = _lib.TsNewKv(_p(k), _p(v), loc, ctypes.pointer(_keep) if pages is not None else None,
                          bt.table.shape[1] * cfg.page_size)
        kv._pool = _keep
        return self._run(q, k_pool, v_pool, bt, out, new_kv=kv)

    def _run(self, q, k_pool, v_pool, bt, out, rerun: bool = False, new_kv=None):
        cfg = self.cfg
        bt = self._options(bt, rerun)
        cb = _c_batch(cfg, bt)
        _need(q, "q", torch.bfloat16, 2)
        rows = q.shape[0]
        if bt.batch != 1 or bt.max_seq_len > self.max_seq_len or rows > self.max_rows:
            raise ValueError("one request, within the sizes this PrefillChunk was built for")
        if q.shape[1] != cfg.num_heads * cfg.head_dim:
            raise ValueError("q must be [rows, H*D]")
        _check_pool(cfg, k_pool, "k_pool")
        _check_pool(cfg, v_pool, "v_pool")
        if out is None:
            out = torch.empty_like(q)
        else:
            _need(out, "out", torch.bfloat16)
            if out.numel() != q.numel():
                raise ValueError("out must hold rows*H*D elements")
        if new_kv is not None:
            _lib.check(_lib.load().ts_prefill_step(
                ctypes.byref(self._c), ctypes.byref(cb), ctypes.byref(new_kv), _p(q), rows, _p(self.cos),
                _p(self.sin), self.cos.shape[0], _p(k_pool), _p(v_pool), k_pool.shape[0], _p(out),
                _p(self.sel), _p(self.sel_pos), cfg.max_sel, _p(self.sel_len), _p(self.workspace),
                self.workspace.numel(), _stream()))
        else:
            _lib.check(_lib.load().ts_prefill_chunk(
                ctypes.byref(self._c), ctypes.byref(cb), _p(q), rows, _p(self.cos), _p(self.sin),
                self.cos.shape[0], _p(k_pool), _p(v_pool), k_pool.shape[0], _p(out), _p(self.sel),
                _p(self.sel_pos), cfg.max_sel, _p(self.sel_len), _p(self.workspace),
                self.workspace.numel(), _stream()))
        return out, self.sel, self.sel_pos, self.sel_len


def sparse_decode_attention_static(cfg: LayerConfig, q: torch.Tensor, k_pool: torch.Tensor,
                                   v_pool: torch.Tensor, sel: torch.Tensor, sel_len: torch.Tensor,
                                   out: torch.Tensor, max_sel_len: Optional[int] = None) -> torch.Tensor:
    """:func:`sparse_decode_attention` through ``ts_sparse_decode_attn_static``: the
    split-K partials live in a buffer built into the library, and neither this wrapper
    nor the library allocates (``out`` [B, H*D] bf16 is the caller's)."""
    c = cfg.to_c()
    _need(q, "q", torch.bfloat16)
    _check_pool(cfg, k_pool, "k_pool")
    _check_pool(cfg, v_pool, "v_pool")
    _need(sel, "sel", torch.int32, 2)
    _need(sel_len, "sel_len", torch.int32, 1)
    _need(out, "out", torch.bfloat16)
    B = sel.shape[0]
    if k_pool.shape != v_pool.shape:
        raise ValueError("k_pool and v_pool must have the same shape")
    if q.numel() != B * cfg.num_heads * cfg.head_dim or sel_len.shape[0] != B or out.numel() != q.numel():
        raise ValueError("q / sel_len / out do not match the batch of sel")
    max_sel_len = sel.shape[1] if max_sel_len is None else int(max_sel_len)
    if max_sel_len > sel.shape[1]:
        raise ValueError("max_sel_len exceeds the width of sel")
    _lib.check(_lib.load().ts_sparse_decode_attn_static(
        ctypes.byref(c), _p(q), _p(k_pool), _p(v_pool), k_pool.shape[0], _p(sel), sel.stride(0),
        _p(sel_len), B, max_sel_len, _p(out), _stream()))
    return out
