"""Oracle (test infrastructure): rotary position embedding.

Follows core/nn/rotary.py of the reference.
"""

from typing import NamedTuple, Optional

import torch


class RotaryTables(NamedTuple):
    cos: torch.Tensor  # [max_seq, dim], module dtype
    sin: torch.Tensor  # [max_seq, dim], module dtype
    dim: int


def rotary_tables(dim: int, max_seq_length: int, base: int = 10000,
                  dtype: torch.dtype = torch.float32) -> RotaryTables:
    """core/nn/rotary.py:93-108 and :149-172.

    inv_freq[i] = base^(-2i/dim) in fp32; angle[p, i] = p * inv_freq[i]; both
    halves of the table hold the same angles; cos/sin are evaluated in fp32 and
    then cast to the module dtype.
    """
    assert dim > 1
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim))
    ang = torch.outer(torch.arange(max_seq_length).float(), inv_freq)
    ang = torch.cat((ang, ang), dim=-1).float()
    return RotaryTables(ang.cos().to(dtype), ang.sin().to(dtype), dim)


def _rotate_half(x: torch.Tensor) -> torch.Tensor:
    """core/nn/rotary.py:111-113."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def _rotate(x: torch.Tensor, position_ids: Optional[torch.Tensor], tables: RotaryTables) -> torch.Tensor:
    # x [s, b, n, dim]; position_ids [s, b] or None (then the table is used row by row)
    if position_ids is None:
        cos = tables.cos[:, None, None, :]
        sin = tables.sin[:, None, None, :]
    else:
        cos = tables.cos[position_ids][:, :, None, :]  # gather of table rows, rotary.py:9-23
        sin = tables.sin[position_ids][:, :, None, :]
    return (x * cos) + (_rotate_half(x) * sin)  # rotary.py:139, arithmetic in x's dtype


def apply_rotary(query: torch.Tensor, key: torch.Tensor, tables: RotaryTables,
                 query_position_ids: Optional[torch.Tensor] = None,
                 key_position_ids: Optional[torch.Tensor] = None):
    """core/nn/rotary.py:117-139 and :176-213.

    query [s_q, b, n_q, d], key [s_k, b, n_kv, d], ids [s, b].  Only the first
    `tables.dim` features rotate (partial rotary, lines 183-203).
    """
    r = tables.dim

    def one(x, ids):
        if x.shape[-1] == r:
            return _rotate(x, ids, tables)
        assert x.shape[-1] > r
        return torch.cat((_rotate(x[..., :r], ids, tables), x[..., r:]), dim=-1)

    return one(query, query_position_ids), one(key, key_position_ids)


def apply_rotary_complex(query: torch.Tensor, key: torch.Tensor, dim: int, max_seq_length: int, base: float,
                         query_position_ids: Optional[torch.Tensor] = None,
                         key_position_ids: Optional[torch.Tensor] = None):
    """core/nn/rotary.py:45-90 and :216-255: interleaved pairs (2i, 2i+1), fp32 math, cast back."""
    inv_freq = 1.0 / (float(base) ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    ang = torch.outer(torch.arange(max_seq_length).float(), inv_freq).float()  # [max_seq, dim/2]

    def one(x, ids):
        s, b, n, d = x.shape
        a = ang[:s][:, None, :].expand(s, b, dim // 2) if ids is None else ang[ids]  # [s, b, dim/2]
        a = a[:, :, None, :]
        xf = x.float().reshape(s, b, n, d // 2, 2)
        re, im = xf[..., 0], xf[..., 1]
        c, sn = a.cos(), a.sin()
        out = torch.stack((re * c - im * sn, re * sn + im * c), dim=-1).reshape(s, b, n, d)
        return out.type_as(x)

    return one(query, query_position_ids), one(key, key_position_ids)
