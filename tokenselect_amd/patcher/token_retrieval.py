"""Host-side mirror of the reference's patch layer and selection runtime
(``patcher/token_retrieval.py``), over the HIP library.

The names, argument order and error behaviour of the reference's entry points
are kept so that a user of the reference can switch imports:

``patch`` tr.py:885-922 · ``RotaryEmbedding`` tr.py:56-114 ·
``ReqToTokenRetriever`` tr.py:117-163 · ``paged_matmul`` tr.py:234-261 ·
``TokenRetriever`` tr.py:264-449 · ``patch_model_runner`` tr.py:452 ·
``patch_input_metadata`` tr.py:475 · ``patch_model`` tr.py:658 and the patched
forwards tr.py:703-866.

What differs, on purpose:

* every tensor operation of the hot path is one call into
  ``libtokenselect_hip.so``; nothing here computes on the CPU and nothing falls
  back to PyTorch ops when the library is missing;
* scores, softmax and votes are fp32 (the reference stores bf16, tr.py:345-347),
  ties in the top-k go to the lowest position;
* the decode forward issues one fused library call per layer (fingerprint,
  selection, sparse attention) and never synchronises with the host, where the
  reference re-plans a FlashInfer wrapper (tr.py:794-813);
* the selection cache works when switched on (``patch(..., query_cache=True)``);
  the reference hard-codes it off and its branch cannot run (tr.py:918, 412).

SGLang and vLLM are optional: when they are importable the same class
attributes the reference overwrites are overwritten; otherwise the duck-typed
classes of :mod:`tokenselect_amd.patcher.sglang_standins` are patched.
"""

from contextlib import contextmanager
from math import ceil
from typing import Optional

import torch

from .. import ops
from . import sglang_standins as _standins

ROPE_BASE = -1
ROPE_SCALE = -1
ROPE_MODE = ""
MAX_N_TOKENS = -1
TOP_K = -1
N_INIT = -1
N_Local = -1
PREFILL_CHUNK_SIZE = -1
QUERY_ROTATE = False
QUERY_CACHE = False
KERNEL_SIZE = -1


@contextmanager
def cuda_timer(timer_name="Operation"):
    """Event timer around a block on the current stream (tr.py:41-53)."""
    torch.cuda.synchronize()
    begin = torch.cuda.Event(enable_timing=True)
    finish = torch.cuda.Event(enable_timing=True)
    begin.record()
    yield
    finish.record()
    torch.cuda.synchronize()
    print(f"{timer_name} time (ms): {begin.elapsed_time(finish):.4f}")


def _mode_name(mode) -> str:
    return getattr(mode, "name", str(mode))


class RotaryEmbedding(torch.nn.Module):
    """tr.py:56-114.  Tables are built with the reference's fp32 torch expressions
    (on the host, then moved to ``device``); the rotation itself is the HIP kernel
    ``ts_rope_apply``, bit-identical to the reference's elementwise expression for
    the same tables."""

    def __init__(self, dim: int, base: float, distance_scale: float = 1.0,
                 device: torch.device = "cuda"):
        super().__init__()
        self.dim = dim
        self.base = base
        self.distance_scale = distance_scale
        self.device = device
        self._seq_len_cached = -1
        self._cos_table = None
        self._sin_table = None

    def _init_inv_freq(self):
        exponent = torch.arange(0, self.dim, 2, dtype=torch.float32) / self.dim
        self.register_buffer("inv_freq", (1.0 / (self.base ** exponent)).to(self.device),
                             persistent=False)

    def _update_cos_sin_tables(self, seq_len: int):
        if not hasattr(self, "inv_freq"):
            self._init_inv_freq()
        if seq_len > self._seq_len_cached:
            self._seq_len_cached = seq_len
            angles = torch.outer(torch.arange(seq_len) * self.distance_scale, self.inv_freq.cpu())
            angles = torch.cat((angles, angles), dim=-1)
            self._cos_table = angles.cos().unsqueeze(1).to(self.device)
            self._sin_table = angles.sin().unsqueeze(1).to(self.device)

    def apply_rotary_pos_emb(self, x: torch.Tensor, position_ids: torch.Tensor,
                             max_position: Optional[int] = None) -> torch.Tensor:
        """``max_position`` lets a caller that knows the largest position avoid the
        host read-back of ``position_ids.max()`` (tr.py:101)."""
        if max_position is None:
            max_position = int(position_ids.max())
        self._update_cos_sin_tables(max_position + 1)
        squeeze = x.dim() == 2
        x3 = x.unsqueeze(1) if squeeze else x
        out = ops.rope_apply(x3.contiguous(), self._cos_table.view(-1, self.dim),
                             self._sin_table.view(-1, self.dim),
                             position_ids.to(torch.int64).contiguous())
        return out.squeeze(1) if squeeze else out

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor) -> torch.Tensor:
        return self.apply_rotary_pos_emb(x, position_ids)

    def rotate_half(self, x: torch.Tensor) -> torch.Tensor:
        half = x.shape[-1] // 2
        return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


class ReqToTokenRetriever:
    """tr.py:117-163: hands out the retriever of the running request and starts a
    fresh one whenever the request id changes."""

    def __init__(self, num_layers, head_dim, num_heads, num_kv_heads, fingerprint_dim,
                 max_num_tokens, token_to_kv_pool, dtype, device):
        self.rope_embedding = RotaryEmbedding(head_dim, ROPE_BASE, ROPE_SCALE, device)
        self.kwargs = dict(num_layers=num_layers, head_dim=head_dim, num_heads=num_heads,
                           num_kv_heads=num_kv_heads, fingerprint_dim=fingerprint_dim,
                           max_num_tokens=max_num_tokens, dtype=dtype, device=device,
                           token_to_kv_pool=token_to_kv_pool, rotary_embedding=self.rope_embedding)
        self.current_req_id = None
        self.current_token_retriever = None

    def get_token_retriever(self, req_id):
        if self.current_req_id != req_id:
            self.current_req_id = req_id
            old = self.current_token_retriever
            if old is not None and QUERY_CACHE:
                old.sync_cache_counters()
                if old.retrieval_count > 0:
                    print("skip_count:", old.skip_count)
                    print("retrieval_count:", old.retrieval_count)
                    print("skip_rate:", old.skip_count / old.retrieval_count)
            self.current_token_retriever = TokenRetriever(**self.kwargs)
        return self.current_token_retriever

    def new_token_retriever(self):
        """A retriever for one more request of a batch (the reference keeps a single one)."""
        return TokenRetriever(**self.kwargs)

    def get_batch_token_retriever(self, req_ids, retrievers=None):
        """The batched twin of ``get_token_retriever``: the ``BatchTokenRetriever`` of the
        running requests ``req_ids``, started afresh (from ``retrievers``, one prefilled
        ``TokenRetriever`` per request) whenever the composition of the batch changes."""
        key = tuple(req_ids)
        if self.current_req_id != key:
            if retrievers is None or len(retrievers) != len(key):
                raise ValueError("a new batch needs one prefilled TokenRetriever per request")
            self.current_req_id = key
            self.current_token_retriever = BatchTokenRetriever(list(retrievers),
                                                               self.kwargs["token_to_kv_pool"])
        return self.current_token_retriever


class BatchTokenRetriever:
    """Several running requests decoded together: the batched twin of ``TokenRetriever``
    (the reference serves one running request, tr.py:130, and starts a fresh retriever
    when the request id changes; a batch is the same thing per request).  Built from the
    retrievers of requests that were prefilled one by one: their token tables and lengths
    are copied once into ``[layers, B, max_tokens]`` / ``[layers, B]`` tensors that the
    library reads as a batch; the K / V pools stay aliased.  The batch lives as long as
    its composition does (``ReqToTokenRetriever.get_batch_token_retriever`` starts a new
    one when the request ids change)."""

    def __init__(self, retrievers, token_to_kv_pool):
        first = retrievers[0]
        self.batch = len(retrievers)
        self.num_layers, self.head_dim = first.num_layers, first.head_dim
        self.num_heads, self.num_kv_heads = first.num_heads, first.num_kv_heads
        self.max_num_tokens, self.dtype, self.device = first.max_num_tokens, first.dtype, first.device
        self.token_fingerprints = first.token_fingerprints
        self._value_buffers = [token_to_kv_pool.get_value_buffer(l) for l in range(first.num_layers)]
        self.token_indices = torch.stack([r.token_indices for r in retrievers], dim=1).contiguous()
        self.num_tokens = [[r.num_tokens[l] for r in retrievers] for l in range(self.num_layers)]
        self._num_tokens_dev = torch.stack([r._num_tokens_dev for r in retrievers], dim=1).contiguous()
        self._threshold_hints = torch.stack([r._threshold_hints for r in retrievers], dim=1).contiguous()
        self._layers = {}
        self._caches = None
        if QUERY_CACHE:
            self._caches = [ops.SelectionCache(
                torch.stack([r.query_fingerprints_cache[l] for r in retrievers]).contiguous(),
                torch.stack([r.topk_indices_cache[l] for r in retrievers]).contiguous(),
                torch.stack([r._cache_len_dev[l] for r in retrievers]).contiguous(),
                torch.stack([r._counters_dev[l] for r in retrievers]).contiguous(),
                first._threshold_host) for l in range(self.num_layers)]

    def _config(self, n_init, n_local, topk, scaling=None, logit_cap=0.0) -> ops.LayerConfig:
        return TokenRetriever._config(self, n_init, n_local, topk, scaling, logit_cap)

    def get_all_tokens(self, layer_id):
        """Per request, as ``TokenRetriever.get_all_tokens``."""
        return [self.token_indices[layer_id, b, : n] for b, n in enumerate(self.num_tokens[layer_id])]

    def _note_appended(self, layer_id, count: int):
        assert count == self.batch, "one new token per running request"
        assert max(self.num_tokens[layer_id]) + 1 <= self.max_num_tokens   # tr.py:334
        self.num_tokens[layer_id] = [n + 1 for n in self.num_tokens[layer_id]]

    def store(self, attn, rows_k, rows_v, loc):
        """store_kv_cache + add_k_cache (tr.py:844-854, 332-336) for one new token per request."""
        layer = attn.layer_id
        cfg = self._config(max(N_INIT, 0), max(N_Local, 0), max(TOP_K, 1))
        ops.kv_store(cfg, rows_k.contiguous(), rows_v.contiguous(), loc.to(torch.int32).contiguous(),
                     self.token_fingerprints[layer], self._value_buffers[layer],
                     self.token_indices[layer], self._num_tokens_dev[layer])
        self._note_appended(layer, loc.shape[0])

    def decode_attention(self, attn, q, k_buffer, v_buffer):
        """One fused library call for a decode layer of the whole batch (tr.py:791-825 per request)."""
        layer_id = attn.layer_id
        cfg = self._config(N_INIT, N_Local, TOP_K, attn.scaling, attn.logit_cap)
        key = (attn.scaling, attn.logit_cap)
        runner = self._layers.get(key)
        if runner is None:
            runner = ops.DecodeLayer(cfg, self.batch, self.max_num_tokens, self.device)
            self._layers[key] = runner
        # The lengths go along on the host too: a batch that is too large for one selection
        # launch is then scored in phases packed by what the requests hold.
        bt = ops.Batch(self._num_tokens_dev[layer_id], self.token_indices[layer_id],
                       max(self.num_tokens[layer_id]),
                       host_seq_lens=torch.tensor(self.num_tokens[layer_id], dtype=torch.int32),
                       hint=self._threshold_hints[layer_id])
        out = torch.empty((self.batch, self.num_heads * self.head_dim), dtype=q.dtype, device=q.device)
        runner(q, k_buffer, v_buffer, bt, self._caches[layer_id] if self._caches else None, out=out)
        return out


def paged_matmul(query, token, indices, scores, num_relevant_tokens, num_heads, num_kv_heads,
                 head_dim, BLOCK_SIZE_TOKENS=128):
    """tr.py:234-261 with the same arguments; ``BLOCK_SIZE_TOKENS`` is accepted and
    ignored (the HIP kernel chooses its own tiling)."""
    ops.paged_matmul(query, token, indices, scores, num_relevant_tokens, num_heads, num_kv_heads,
                     head_dim)


class TokenRetriever:
    """tr.py:264-449: per-request, per-layer logical->physical token table and the
    selection over it."""

    def __init__(self, num_layers, head_dim, num_heads, num_kv_heads, fingerprint_dim,
                 max_num_tokens, dtype, device, token_to_kv_pool=None,
                 rotary_embedding: Optional["RotaryEmbedding"] = None):
        self.num_layers = num_layers
        self.head_dim = head_dim
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.fingerprint_dim = fingerprint_dim
        self.max_num_tokens = max_num_tokens
        self.dtype = dtype
        self.device = device
        # K buffers of the host framework, aliased, never copied (tr.py:288-291).
        self.token_fingerprints = [token_to_kv_pool.get_key_buffer(l) for l in range(num_layers)]
        self.token_indices = torch.empty((num_layers, max_num_tokens), device=device,
                                         dtype=torch.int32)
        self.rope_embedding = rotary_embedding
        top_k = max(int(TOP_K), 1)
        self.query_fingerprints_cache = torch.zeros((num_layers, num_heads * head_dim),
                                                    device=device, dtype=dtype)
        # int32 here (the reference keeps int64, tr.py:307-311): positions fit and
        # the library's tables are 32-bit.
        self.topk_indices_cache = torch.zeros((num_layers, top_k), device=device, dtype=torch.int32)
        self.similarity_threshold = torch.tensor([0.9] * num_layers, device=device, dtype=dtype)
        self._threshold_host = float(torch.tensor(0.9, dtype=dtype))  # 0.8984375 in bf16
        self.skip_count = 0
        self.retrieval_count = 0
        self.is_first_query = [True] * num_layers
        # Device-side twins of the host bookkeeping, read by the kernels.
        self._num_tokens_dev = torch.zeros((num_layers,), device=device, dtype=torch.int32)
        self._cache_len_dev = torch.zeros((num_layers,), device=device, dtype=torch.int32)
        self._counters_dev = torch.zeros((num_layers, 2), device=device, dtype=torch.int64)
        # Where the k-th vote of a layer's last selection lay: the single-launch selection's
        # guess for the next step (ts_batch.threshold_hint), one word per layer.
        self._threshold_hints = torch.zeros((num_layers,), device=device, dtype=torch.int32)
        self._layers = {}
        self.clear()

    # ------------------------------------------------------------ bookkeeping
    def clear(self):
        self.num_tokens = [0] * self.num_layers
        self.is_first_query = [True] * self.num_layers
        self.skip_count = 0
        self._num_tokens_dev.zero_()
        self._cache_len_dev.zero_()
        self._counters_dev.zero_()
        self._threshold_hints.zero_()

    def get_all_tokens(self, layer_id):
        return self.token_indices[layer_id, : self.num_tokens[layer_id]]

    def add_k_cache(self, indices, layer_id):
        tail_idx = self.num_tokens[layer_id] + indices.shape[0]
        assert tail_idx <= self.max_num_tokens
        self.token_indices[layer_id, self.num_tokens[layer_id]: tail_idx] = indices
        self.num_tokens[layer_id] = tail_idx
        self._num_tokens_dev[layer_id] = tail_idx

    def _note_appended(self, layer_id, count: int):
        """Host twin of an append the library already did on the device."""
        tail_idx = self.num_tokens[layer_id] + count
        assert tail_idx <= self.max_num_tokens
        self.num_tokens[layer_id] = tail_idx

    def sync_cache_counters(self):
        """Reads the device hit / call counters back (the only host sync of the
        selection cache; the reference counts on the host, tr.py:420-421)."""
        totals = self._counters_dev.sum(dim=0).tolist()
        self.skip_count, self.retrieval_count = int(totals[0]), int(totals[1])

    # --------------------------------------------------------------- selection
    def _config(self, n_init, n_local, topk, scaling=None, logit_cap=0.0) -> ops.LayerConfig:
        return ops.LayerConfig(
            num_heads=self.num_heads, num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
            page_size=1, n_init=n_init, n_local=n_local, top_k=topk, pool_kernel=KERNEL_SIZE,
            head_map="mod", rope_mode=ROPE_MODE if ROPE_MODE else "NONE", rope_theta=float(ROPE_BASE),
            rope_scale=float(ROPE_SCALE), sm_scale=scaling, logit_cap=float(logit_cap or 0.0))

    def get_topk_tokens(self, query_fingerprints, token_fingerprints, topk, indices):
        """tr.py:338-373: positions (ascending, int64, relative to ``indices``) of the
        ``topk`` candidates with the largest soft vote."""
        n = indices.shape[0]
        if topk > n:
            raise RuntimeError("selected index k out of range")
        cfg = self._config(0, 0, topk)
        seq = torch.tensor([n], dtype=torch.int32, device=indices.device)
        bt = ops.Batch(seq, indices.to(torch.int32).contiguous().view(1, -1), n)
        if topk == n:
            return torch.arange(n, device=indices.device)
        scores, partials = ops.score(cfg, bt, query_fingerprints.contiguous(), token_fingerprints)
        votes, _ = ops.vote(cfg, bt, scores, partials)
        _, sel_pos, _ = ops.topk_ragged(cfg, bt, votes)
        return sel_pos[0, :topk].to(torch.int64)

    def _fingerprint(self, query):
        """tr.py:380-392: rotate row i to position n_local + i, average the rows."""
        rows = query.shape[0]
        if rows != 1:
            if not QUERY_ROTATE:
                return query.mean(dim=0, keepdim=True)
            cos, sin = self._rope_tables(rows)
            cfg = self._config(N_INIT, N_Local, TOP_K)
            return ops.fingerprint(cfg, query.view(rows, -1, self.head_dim).contiguous(), cos,
                                   sin).view(1, -1)
        if QUERY_ROTATE:
            # Decode row i sits at position n_local + i (tr.py:381-385); one row -> n_local.
            pos = int(N_Local)
            position_ids = torch.full((1,), pos, device=query.device, dtype=torch.int64)
            return self.rope_embedding.apply_rotary_pos_emb(
                query.view(1, -1, self.head_dim), position_ids, max_position=pos).view(1, -1)
        return query.view(1, -1)

    def _rope_tables(self, rows):
        """cos / sin rows 0 .. n_local + rows - 1 (tr.py:92-96), cached."""
        need = int(N_Local) + rows
        tables = getattr(self, "_tables", None)
        if tables is None or tables[0].shape[0] < need:
            tables = ops.rope_tables(self.head_dim, ROPE_BASE, ROPE_SCALE,
                                     max(need, int(N_Local) + max(PREFILL_CHUNK_SIZE, 1)),
                                     self.device)
            self._tables = tables
        return tables

    def _cache(self, layer_id) -> Optional[ops.SelectionCache]:
        if not QUERY_CACHE:
            return None
        return ops.SelectionCache(
            self.query_fingerprints_cache[layer_id:layer_id + 1],
            self.topk_indices_cache[layer_id:layer_id + 1],
            self._cache_len_dev[layer_id:layer_id + 1],
            self._counters_dev[layer_id:layer_id + 1],
            self._threshold_host)

    def retrieval_indices(self, query, layer_id, n_init, n_local, topk):
        """tr.py:375-449: physical slots ``[n_init + topk + n_local]`` int32 to attend
        to, or ``None`` when the context is too short to select from."""
        current_num_tokens = self.num_tokens[layer_id]
        if n_init + topk + n_local >= current_num_tokens:
            return None
        if n_local != N_Local and QUERY_ROTATE:
            raise ValueError("the query is rotated to the patched N_Local; pass n_local == N_Local")
        cfg = self._config(n_init, n_local, topk)
        qf = self._fingerprint(query)
        bt = ops.Batch(self._num_tokens_dev[layer_id:layer_id + 1],
                       self.token_indices[layer_id:layer_id + 1], current_num_tokens,
                       hint=self._threshold_hints[layer_id:layer_id + 1] if query.shape[0] == 1 else None)
        cache = self._cache(layer_id)
        k_buffer = self.token_fingerprints[layer_id]
        # The large buffers are kept between calls, sized for the longest table.
        key = ("select", n_init, n_local, topk, KERNEL_SIZE)
        sized = ops.Batch(bt.seq_lens, bt.table, self.max_num_tokens)
        one_launch = not getattr(self, "_separate", False) and \
            ops.select_supported(cfg, 1, self.max_num_tokens)
        held = self._layers.get(key)
        if one_launch and held is not None and ops.gave_up(held[1]):
            # An earlier launch gave up and nobody noticed at a synchronisation point: what it
            # selected was not valid.  From now on the separate kernels, whose workgroups never
            # wait for each other; the caller retries the request.
            self._separate = True
            del self._layers[key]
            raise ops.SelectionGaveUp(
                "the single-launch selection gave up waiting for its workgroups (another stream "
                "or process on the GPU?): the selection of an earlier call was not valid; this "
                "retriever now uses the separate kernels, retry the request")
        hit = ops.selcache_step(cfg, bt, qf, cache) if cache is not None else None
        if one_launch:
            # the whole selection in one launch
            if held is None:
                held = (ops.select_workspace(cfg, sized, self.device), ops.fault_word())
                self._layers[key] = held
            workspace, fault = held
            bt.fault = fault
            sel, _, _, _, _ = ops.select(cfg, bt, qf, k_buffer, hit=hit, cache=cache,
                                         workspace=workspace)
        else:
            if held is None:
                held = ops.score_buffers(cfg, sized, self.device)
                self._layers[key] = held
            scores, partials = ops.score(cfg, bt, qf, k_buffer, skip=hit, out=held)
            votes, _ = ops.vote(cfg, bt, scores, partials, skip=hit)
            sel, _, _ = ops.topk_ragged(cfg, bt, votes, hit=hit, cache=cache)
        if cache is not None:
            self.is_first_query[layer_id] = False
        return sel[0, : n_init + topk + n_local]

    # ------------------------------------------------------- fused decode step
    def decode_attention(self, attn, q, k_buffer, v_buffer):
        """One fused library call for a decode layer: selection (or the dense
        fallback) and the attention over the result (tr.py:791-825)."""
        layer_id = attn.layer_id
        cfg = self._config(N_INIT, N_Local, TOP_K, attn.scaling, attn.logit_cap)
        key = (attn.scaling, attn.logit_cap)
        runner = self._layers.get(key)
        if runner is None:
            runner = ops.DecodeLayer(cfg, 1, self.max_num_tokens, self.device)
            self._layers[key] = runner
        bt = ops.Batch(self._num_tokens_dev[layer_id:layer_id + 1],
                       self.token_indices[layer_id:layer_id + 1], self.num_tokens[layer_id],
                       hint=self._threshold_hints[layer_id:layer_id + 1])
        out = torch.empty((1, self.num_heads * self.head_dim), dtype=q.dtype, device=q.device)
        cache = self._cache(layer_id)
        runner(q, k_buffer, v_buffer, bt, cache, out=out)
        if cache is not None:
            self.is_first_query[layer_id] = False
        return out


    # ------------------------------------------------------ fused prefill chunk
    def prefill_attention(self, attn, q, k_buffer, v_buffer):
        """One fused library call for a prefill chunk after its KV store: chunk
        fingerprint, selection (or the dense fallback) and the causal attention of the
        chunk's rows over the result (tr.py:735-773)."""
        layer_id = attn.layer_id
        cfg = self._config(N_INIT, N_Local, TOP_K, attn.scaling, attn.logit_cap)
        key = ("prefill", attn.scaling, attn.logit_cap)
        runner = self._layers.get(key)
        if runner is None:
            runner = ops.PrefillChunk(cfg, self.max_num_tokens, self.device,
                                      max_rows=max(PREFILL_CHUNK_SIZE, 1))
            self._layers[key] = runner
        bt = ops.Batch(self._num_tokens_dev[layer_id:layer_id + 1],
                       self.token_indices[layer_id:layer_id + 1], self.num_tokens[layer_id])
        out, _, _, _ = runner(q, k_buffer, v_buffer, bt)
        return out


# ----------------------------------------------------------- patched forwards
def patched_radix_attention_store_kv_cache(self, cache_k, cache_v, input_metadata, start=0, end=None):
    """tr.py:844-854: scatter the new K/V rows into the pool and append their slots
    to the request's table - one fused kernel for a decode row or a prefill chunk."""
    k_cache = input_metadata.token_to_kv_pool.get_key_buffer(self.layer_id)
    v_cache = input_metadata.token_to_kv_pool.get_value_buffer(self.layer_id)
    loc = input_metadata.out_cache_loc[start:end]
    retriever = input_metadata.token_retriever
    rows_k, rows_v = cache_k[start:end], cache_v[start:end]
    if isinstance(retriever, BatchTokenRetriever):
        retriever.store(self, rows_k, rows_v, loc)
        return
    if loc.dtype == torch.int32 and loc.shape[0] >= 1:
        cfg = retriever._config(max(N_INIT, 0), max(N_Local, 0), max(TOP_K, 1))
        layer = self.layer_id
        if loc.shape[0] == 1:
            ops.kv_store(cfg, rows_k.contiguous(), rows_v.contiguous(), loc.contiguous(), k_cache,
                         v_cache, retriever.token_indices[layer:layer + 1],
                         retriever._num_tokens_dev[layer:layer + 1])
        else:
            assert retriever.num_tokens[layer] + loc.shape[0] <= retriever.max_num_tokens
            ops.kv_store_chunk(cfg, rows_k.contiguous(), rows_v.contiguous(), loc.contiguous(),
                               k_cache, v_cache, retriever.token_indices[layer],
                               retriever._num_tokens_dev[layer:layer + 1])
        retriever._note_appended(layer, loc.shape[0])
        return
    k_cache[loc] = rows_k
    v_cache[loc] = rows_v
    retriever.add_k_cache(loc, self.layer_id)


def patched_radix_attention_decode_forward_flashinfer(self, q, k, v, input_metadata):
    """tr.py:777-825 without FlashInfer: store, select, attend."""
    if self.sliding_window_size != -1:
        raise NotImplementedError("Sliding window not supported yet")
    if k is not None:
        assert v is not None
        self.store_kv_cache(k, v, input_metadata)
    batched = isinstance(input_metadata.token_retriever, BatchTokenRetriever)
    if q.shape[0] != (input_metadata.token_retriever.batch if batched else 1):
        raise NotImplementedError(
            "the patched decode forward serves one running request, as the reference does "
            "(tr.py:130), or the requests of a BatchTokenRetriever "
            "(ReqToTokenRetriever.get_batch_token_retriever)")
    k_buffer, v_buffer = input_metadata.token_to_kv_pool.get_kv_buffer(self.layer_id)
    o = input_metadata.token_retriever.decode_attention(self, q.contiguous(), k_buffer, v_buffer)
    return o.view(-1, self.tp_q_head_num * self.head_dim)


def patched_radix_attention_extend_forward_flashinfer(self, q, k, v, input_metadata):
    """tr.py:703-775 without FlashInfer: the prompt in chunks of PREFILL_CHUNK_SIZE rows;
    per chunk store its K/V, select once for the whole chunk, attend causally."""
    if self.sliding_window_size != -1:
        raise NotImplementedError("Sliding window not supported yet")
    assert not getattr(input_metadata, "flashinfer_use_ragged", False)  # not supported yet
    num_chunks = ceil(q.shape[0] / PREFILL_CHUNK_SIZE)
    outputs = torch.empty_like(q)
    k_buffer, v_buffer = input_metadata.token_to_kv_pool.get_kv_buffer(self.layer_id)
    for chunk_idx in range(num_chunks):
        start = chunk_idx * PREFILL_CHUNK_SIZE
        end = min((chunk_idx + 1) * PREFILL_CHUNK_SIZE, q.shape[0])
        if k is not None:
            assert v is not None
            self.store_kv_cache(k, v, input_metadata, start=start, end=end)
        o = input_metadata.token_retriever.prefill_attention(
            self, q[start:end].contiguous().view(end - start, -1), k_buffer, v_buffer)
        outputs[start:end] = o.view(end - start, -1)
    return outputs


def patched_radix_attention_forward(self, q, k, v, input_metadata):
    """tr.py:827-842."""
    if k is not None:
        assert v is not None
        k = k.view(-1, self.tp_k_head_num, self.qk_head_dim)
        v = v.view(-1, self.tp_v_head_num, self.v_head_dim)
    mode = _mode_name(input_metadata.forward_mode)
    if mode == "EXTEND":
        return patched_radix_attention_extend_forward_flashinfer(self, q, k, v, input_metadata)
    elif mode == "DECODE":
        return patched_radix_attention_decode_forward_flashinfer(self, q, k, v, input_metadata)


def patched_meta_attention_forward(self, positions, hidden_states, input_metadata):
    """tr.py:856-866: QKV projection, attention WITHOUT the model's rotary
    embedding (K stays un-rotated in the cache), output projection."""
    qkv, _ = self.qkv_proj(hidden_states)
    q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
    attn_output = self.attn(q, k, v, input_metadata)
    output, _ = self.o_proj(attn_output)
    return output


def patch_attention(model):
    """tr.py:868-876: overwrite the class-level forwards of every layer's
    attention module and of its ``RadixAttention``."""
    for layer in model.model.layers:
        layer.self_attn.__class__.forward = patched_meta_attention_forward
        layer.self_attn.attn.__class__.forward = patched_radix_attention_forward
        layer.self_attn.attn.__class__.store_kv_cache = patched_radix_attention_store_kv_cache
    return model


def _sglang():
    try:
        import sglang  # noqa: F401
        import sglang.srt.model_executor.model_runner as model_runner
        import sglang.srt.model_executor.forward_batch_info as forward_batch_info
        return model_runner, forward_batch_info
    except ImportError:
        return None


def patch_model_runner():
    """tr.py:452-472: a ``ModelRunner`` that owns the ``ReqToTokenRetriever``."""
    found = _sglang()
    base = found[0].ModelRunner if found else _standins.BASE_MODEL_RUNNER

    class PatchedModelRunner(base):
        def __init__(self, **kwargs):
            super().__init__(**kwargs)
            kv_heads = self.model_config.get_num_kv_heads(self.tp_size)
            self.req_to_token_retriever = ReqToTokenRetriever(
                self.model_config.num_hidden_layers, self.model_config.head_dim,
                self.model_config.num_attention_heads, kv_heads,
                kv_heads * self.model_config.head_dim, MAX_N_TOKENS, self.token_to_kv_pool,
                self.dtype, "cuda")
            print("max_total_num_tokens:", self.max_total_num_tokens)

    if found:
        found[0].ModelRunner = PatchedModelRunner
    else:
        _standins.ModelRunner = PatchedModelRunner
    return PatchedModelRunner


def patch_input_metadata():
    """tr.py:475-655: the step metadata carries the running request's retriever.
    The FlashInfer index planning the reference redoes here (tr.py:570-650) has no
    counterpart: the library plans its split-K schedule on the device."""
    found = _sglang()
    if not found:
        return _standins.InputMetadata  # already carries token_retriever
    base = found[1].InputMetadata

    class PatchedInputMetadata(base):
        token_retriever: TokenRetriever

        def __init__(self, **kwargs):
            self.token_retriever = kwargs.pop("token_retriever")
            super().__init__(**kwargs)

        def init_flashinfer_handlers(self, model_runner, prefix_lens, flashinfer_use_ragged):
            self.flashinfer_use_ragged = False

        @classmethod
        def from_schedule_batch(cls, model_runner, batch, forward_mode):
            ret = cls(
                forward_mode=forward_mode, batch_size=batch.batch_size(),
                req_pool_indices=batch.req_pool_indices, seq_lens=batch.seq_lens,
                req_to_token_pool=model_runner.req_to_token_pool,
                token_to_kv_pool=model_runner.token_to_kv_pool,
                token_retriever=model_runner.req_to_token_retriever.get_token_retriever(
                    batch.reqs[0].rid),
                out_cache_loc=batch.out_cache_loc, return_logprob=batch.return_logprob,
                top_logprobs_nums=batch.top_logprobs_nums)
            ret.compute_positions(batch)
            ret.compute_extend_infos(batch)
            if _mode_name(forward_mode) != "DECODE":
                ret.total_num_tokens = int(torch.sum(ret.seq_lens))
                ret.init_multimuldal_info(batch)
            ret.init_flashinfer_handlers(model_runner, None, False)
            return ret

    found[1].InputMetadata = PatchedInputMetadata
    found[1].update_flashinfer_indices = patched_forward_batch_info_update_flashinfer_indices
    return PatchedInputMetadata


def patched_forward_batch_info_update_flashinfer_indices(
        forward_mode, model_runner, req_pool_indices, seq_lens, prefix_lens,
        flashinfer_decode_wrapper=None, flashinfer_use_ragged=False):
    """Stands in for the function the reference installs as
    ``forward_batch_info.update_flashinfer_indices`` (tr.py:570-655), with its signature
    and the configurations it refuses (tr.py:589, 635, 650).  The reference rebuilds the
    dense ``kv_indptr`` / ``kv_indices`` on the host here and re-plans the FlashInfer
    wrappers; the library plans its split-K schedule on the device from ``sel_len``, so
    nothing is left to do."""
    if getattr(model_runner, "sliding_window_size", None) is not None:
        raise NotImplementedError("Sliding window not supported yet")
    if flashinfer_use_ragged:
        raise NotImplementedError("Ragged attention not supported yet")
    return None


def patch_model():
    """tr.py:658-882: models lose their rotary embedding and get the patched
    attention forwards.  With vLLM present its loader is wrapped the way the
    reference does; otherwise the stand-in classes are patched directly."""
    try:
        from vllm.model_executor.layers import rotary_embedding
        from vllm.model_executor.model_loader.loader import DefaultModelLoader
    except ImportError:
        _standins.Attention.forward = patched_meta_attention_forward
        _standins.RadixAttention.forward = patched_radix_attention_forward
        _standins.RadixAttention.store_kv_cache = patched_radix_attention_store_kv_cache
        return

    original_load = DefaultModelLoader.load_model

    def patched_default_model_loader_load_model(self, **kwargs):
        return patch_attention(original_load(self, **kwargs))

    def patched_rotary_embedding_get_rope(*args, **kwargs) -> None:
        return None

    rotary_embedding.get_rope = patched_rotary_embedding_get_rope
    DefaultModelLoader.load_model = patched_default_model_loader_load_model


def patch(rope_base=1e6, rope_scale=1, rope_model="ROPE_LLAMA", max_n_tokens=1024, top_k=16,
          n_init=1, n_local=16, kernel_size=-1, *, query_cache=False):
    """tr.py:885-922.  ``query_cache`` is an addition (keyword only): the reference
    hard-codes ``QUERY_CACHE = False`` (tr.py:918)."""
    global ROPE_BASE, ROPE_SCALE, ROPE_MODE, MAX_N_TOKENS, TOP_K, N_INIT, N_Local
    global QUERY_ROTATE, QUERY_CACHE, PREFILL_CHUNK_SIZE, KERNEL_SIZE

    ROPE_BASE = rope_base
    ROPE_SCALE = rope_scale
    ROPE_MODE = rope_model
    MAX_N_TOKENS = max_n_tokens
    TOP_K = top_k
    N_INIT = n_init
    N_Local = n_local
    KERNEL_SIZE = kernel_size

    QUERY_ROTATE = True
    PREFILL_CHUNK_SIZE = 512
    QUERY_CACHE = bool(query_cache)

    patch_input_metadata()
    patch_model_runner()
    patch_model()
