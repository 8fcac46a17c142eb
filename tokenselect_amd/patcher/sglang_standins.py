"""Duck-typed stand-ins for the SGLang 0.2.13 objects the patch layer touches.

SGLang / vLLM are not importable where this library is built and measured, so
the patched forwards are exercised against these minimal classes.  They carry
exactly the attributes the reference reads (``patcher/token_retrieval.py``):
off ``RadixAttention`` ``layer_id, tp_q_head_num, tp_k_head_num, tp_v_head_num,
head_dim, qk_head_dim, v_head_dim, scaling, logit_cap, sliding_window_size``
(tr.py:708, 754-756, 768, 781, 816-819, 832-833); off ``InputMetadata``
``forward_mode, token_retriever, token_to_kv_pool, out_cache_loc`` (tr.py:780,
791, 817, 835, 847-852); off the attention module ``qkv_proj, o_proj, q_size,
kv_size, attn`` (tr.py:862-865).
"""

import enum
from dataclasses import dataclass
from typing import Any, Optional

import torch


class ForwardMode(enum.IntEnum):
    PREFILL = 1
    EXTEND = 2
    DECODE = 3


class TokenToKVPool:
    """Per-layer K and V buffers ``[size + 1, Hkv, D]`` (SGLang's MHATokenToKVPool)."""

    def __init__(self, size: int, dtype, head_num: int, head_dim: int, layer_num: int, device):
        self.size = size
        self.k_buffer = [torch.zeros((size + 1, head_num, head_dim), dtype=dtype, device=device)
                         for _ in range(layer_num)]
        self.v_buffer = [torch.zeros((size + 1, head_num, head_dim), dtype=dtype, device=device)
                         for _ in range(layer_num)]

    def get_key_buffer(self, layer_id: int):
        return self.k_buffer[layer_id]

    def get_value_buffer(self, layer_id: int):
        return self.v_buffer[layer_id]

    def get_kv_buffer(self, layer_id: int):
        return self.k_buffer[layer_id], self.v_buffer[layer_id]


@dataclass
class InputMetadata:
    forward_mode: ForwardMode
    token_retriever: Any
    token_to_kv_pool: TokenToKVPool
    out_cache_loc: torch.Tensor
    batch_size: int = 1
    flashinfer_decode_wrapper: Any = None
    flashinfer_prefill_wrapper_paged: Any = None
    flashinfer_use_ragged: bool = False


class RadixAttention(torch.nn.Module):
    def __init__(self, num_heads: int, head_dim: int, scaling: float, num_kv_heads: int,
                 layer_id: int, sliding_window_size: int = -1, logit_cap: float = -1):
        super().__init__()
        self.tp_q_head_num = num_heads
        self.tp_k_head_num = num_kv_heads
        self.tp_v_head_num = num_kv_heads
        self.head_dim = head_dim
        self.qk_head_dim = head_dim
        self.v_head_dim = head_dim
        self.scaling = scaling
        self.layer_id = layer_id
        self.sliding_window_size = sliding_window_size
        self.logit_cap = logit_cap if logit_cap is not None and logit_cap > 0 else 0

    def forward(self, q, k, v, input_metadata):  # replaced by patch_model()
        raise RuntimeError("RadixAttention.forward was not patched: call patch() first")

    def store_kv_cache(self, cache_k, cache_v, input_metadata, start=0, end=None):
        raise RuntimeError("RadixAttention.store_kv_cache was not patched: call patch() first")


class _TupleLinear(torch.nn.Linear):
    """vLLM's parallel linear layers return ``(output, bias)``."""

    def forward(self, x):  # type: ignore[override]
        return super().forward(x), None


class Attention(torch.nn.Module):
    """The model's attention module (LlamaAttention / Qwen2Attention shape)."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 layer_id: int, dtype=torch.bfloat16, device=None, bias: bool = False):
        super().__init__()
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        self.qkv_proj = _TupleLinear(hidden_size, self.q_size + 2 * self.kv_size, bias=bias,
                                     dtype=dtype, device=device)
        self.o_proj = _TupleLinear(self.q_size, hidden_size, bias=False, dtype=dtype, device=device)
        self.attn = RadixAttention(num_heads, head_dim, head_dim ** -0.5, num_kv_heads, layer_id)

    def forward(self, positions, hidden_states, input_metadata):  # replaced by patch_model()
        raise RuntimeError("attention forward was not patched: call patch() first")


@dataclass
class ModelConfig:
    num_hidden_layers: int
    head_dim: int
    num_attention_heads: int
    num_key_value_heads: int

    def get_num_kv_heads(self, tp_size: int) -> int:
        return max(1, self.num_key_value_heads // tp_size)


class ModelRunner:
    """The few ModelRunner members ``PatchedModelRunner`` reads (tr.py:455-470)."""

    def __init__(self, model_config: ModelConfig, token_to_kv_pool: TokenToKVPool, dtype,
                 tp_size: int = 1, max_total_num_tokens: Optional[int] = None):
        self.model_config = model_config
        self.token_to_kv_pool = token_to_kv_pool
        self.dtype = dtype
        self.tp_size = tp_size
        self.max_total_num_tokens = max_total_num_tokens or token_to_kv_pool.size


BASE_MODEL_RUNNER = ModelRunner  # patch_model_runner() subclasses this, however often it runs
