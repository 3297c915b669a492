"""Rotary position embedding, CPU restatement (TEST INFRASTRUCTURE, not product code).

Follows ironcore/layers/positional_embedding/rotary.py:

* ``rope_tables``  = the cached tables of ``__init__`` / ``_update_rope_cache``
  (rotary.py:31-51): theta_i = base^(-2i/hd), angle = (offset + p) * scale *
  theta_i, fp32 sin and cos.
* ``rope_rotate``  = ``apply_rotary_pos_emb`` (rotary.py:69-83), same torch ops
  in the same order: pairs (x[2i], x[2i+1]), ``x1*cos - x2*sin`` and
  ``x1*sin + x2*cos`` with the fp32 tables (so the arithmetic is fp32 by type
  promotion and the result is fp32, as in the reference), re-interleaved.

What differs from the reference on purpose: WHICH table row a token uses is an
explicit argument, ``positions``.  The reference's ``forward`` transposes its
input to [s, b, h, d] and then slices the tables by ``x.size(1)`` (rotary.py:
55-64), so the angle of a row is chosen by its BATCH index; ``positions =
batch index`` reproduces that, ``positions = index in the sequence`` is what a
KV-cached decoder needs.

Pinned by (tests/test_oracle_rope.py): complex multiplication in float64
((x1 + i x2) * exp(i angle)), position 0 == identity bit for bit, pair norms
preserved, <rope(q, m), rope(k, n)> a function of m - n only, tables against
float64 closed forms.  The reference's tests hold shape checks only for it.
"""
from __future__ import annotations

import torch


def rope_tables(head_dim: int, max_positions: int, base: float = 10000, scale: float = 1.0,
                offset: int = 0):
    """(cos, sin), each fp32 [max_positions, head_dim // 2] (rotary.py:31-51)."""
    theta = 1.0 / (base ** (torch.arange(0, head_dim, 2).float() / head_dim))
    position = torch.arange(offset, offset + max_positions, dtype=torch.float32)
    position *= scale
    idx_theta = torch.einsum("i,j->ij", position, theta)
    return torch.cos(idx_theta), torch.sin(idx_theta)


def rope_rotate(x: torch.Tensor, positions: torch.Tensor, cos_table: torch.Tensor,
                sin_table: torch.Tensor) -> torch.Tensor:
    """x [n, heads, hd], positions [n] -> rotated rows, fp32 (rotary.py:69-83)."""
    cos_emb = cos_table[positions.long()].unsqueeze(1)  # [n, 1, hd/2], broadcast over heads
    sin_emb = sin_table[positions.long()].unsqueeze(1)
    x1 = x[..., ::2]
    x2 = x[..., 1::2]
    x_rotated = torch.stack([x1 * cos_emb - x2 * sin_emb, x1 * sin_emb + x2 * cos_emb], dim=-1)
    return x_rotated.flatten(-2)
