"""Oracle: rotary embedding of the scoring query (test infrastructure only).

Follows ``patcher/token_retrieval.py:56-114`` (``RotaryEmbedding``):
inverse frequencies tr.py:75-81, tables tr.py:92-96, application tr.py:102-107,
``rotate_half`` tr.py:112-114.
"""

import torch


def inv_freq(dim: int, base: float) -> torch.Tensor:
    """``1 / base^(2i/dim)`` for i in [0, dim/2), fp32 (tr.py:75-81)."""
    exponent = torch.arange(0, dim, 2, dtype=torch.float32) / dim
    return 1.0 / (base ** exponent)


def cos_sin_tables(seq_len: int, dim: int, base: float, distance_scale=1.0):
    """fp32 tables of shape ``[seq_len, 1, dim]`` (tr.py:92-96).

    The angle of column ``i`` and of column ``i + dim/2`` is the same:
    ``position * distance_scale * inv_freq[i]``.
    """
    positions = torch.arange(seq_len)
    angles = torch.outer(positions * distance_scale, inv_freq(dim, base))
    angles = torch.cat((angles, angles), dim=-1)
    return angles.cos().unsqueeze(1), angles.sin().unsqueeze(1)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """``(x1, x2) -> (-x2, x1)`` over the last dimension (tr.py:112-114)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply(x: torch.Tensor, position_ids: torch.Tensor, base: float,
          distance_scale=1.0) -> torch.Tensor:
    """Rotate ``x`` of shape ``[rows, heads, dim]`` to ``position_ids[rows]``.

    fp32 arithmetic, result cast back to ``x.dtype`` (tr.py:98-107).
    """
    dim = x.shape[-1]
    cos, sin = cos_sin_tables(int(position_ids.max()) + 1, dim, base, distance_scale)
    c = cos[position_ids]
    s = sin[position_ids]
    return (x.float() * c + rotate_half(x).float() * s).to(x.dtype)


def scoring_query(q: torch.Tensor, num_heads: int, head_dim: int, n_local: int,
                  base: float, distance_scale=1.0) -> torch.Tensor:
    """Fingerprint of a decode query: rotate row ``i`` to ``n_local + i`` and
    average over the rows (tr.py:380-392).  ``q`` is ``[rows, heads*dim]``;
    returns ``[heads*dim]`` in ``q.dtype``."""
    rows = q.shape[0]
    position_ids = torch.arange(n_local, n_local + rows)
    rotated = apply(q.view(rows, num_heads, head_dim), position_ids, base, distance_scale)
    return torch.mean(rotated.view(rows, -1), dim=0)
