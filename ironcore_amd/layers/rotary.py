"""Rotary position embedding: mirror of the reference module
(ironcore/layers/positional_embedding/rotary.py:15-83) on the HIP kernel.

Same constructor, same buffers (``theta``, ``sin_emb``, ``cos_emb``), same
rotation of the element pairs (2i, 2i+1).  Two differences, both deliberate:

* ``forward(x, positions=None)`` takes the table row of every token as an
  optional argument.  Without it the module does what the reference does:
  after its transpose the reference slices the tables by ``x.size(1)``, which
  is the BATCH size (rotary.py:55-64), so the angle of a row is chosen by its
  batch index.  A KV-cached decoder passes each token's index in its sequence.
* The result has the dtype of ``x``.  The reference multiplies by its fp32
  tables and so returns fp32 by type promotion; here the same fp32 arithmetic
  is rounded once to the element type, which is what reaches a 16-bit KV
  cache anyway.

In the cached path the rotation is fused into the KV append
(``paged_ops.rope_kv_append``); this module then only lends its tables.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import paged_ops


class RotaryPositionalEmbedding(nn.Module):
    def __init__(self, head_dim: int, max_seq_len: int = 4096, base: int = 10000, scale: float = 1.0,
                 offset: int = 0):
        super().__init__()
        self.head_dim = head_dim
        self.max_seq_len = max_seq_len
        self.rope_base = base
        self.offset = offset
        self.scale = scale
        theta = 1.0 / (base ** (torch.arange(0, head_dim, 2).float() / head_dim))
        self.register_buffer("theta", theta)
        self._update_rope_cache(max_seq_len)

    def _update_rope_cache(self, max_seq_len: int) -> None:
        """rotary.py:36-51: fp32 sin/cos of (offset + p) * scale * theta_i."""
        self.max_seq_len_cached = max_seq_len
        position = torch.arange(self.offset, self.offset + max_seq_len, dtype=torch.float32,
                                device=self.theta.device)
        position *= self.scale
        idx_theta = torch.einsum("i,j->ij", position, self.theta)
        self.register_buffer("sin_emb", torch.sin(idx_theta).contiguous(), persistent=False)
        self.register_buffer("cos_emb", torch.cos(idx_theta).contiguous(), persistent=False)

    def _apply(self, fn, recurse=True):
        """``model.to(torch.bfloat16)`` would round the tables (module buffers)
        to 16 bits; the angles are fp32 by construction (rotary.py:31-51), so
        a dtype change rebuilds them in fp32 on whatever device they moved to."""
        super()._apply(fn, recurse)
        if self.theta.dtype != torch.float32:
            device = self.theta.device
            self.theta = 1.0 / (self.rope_base ** (torch.arange(0, self.head_dim, 2, device=device).float()
                                                   / self.head_dim))
            self._update_rope_cache(self.max_seq_len_cached)
        return self

    def forward(self, x: torch.Tensor, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x`` ``[b, s, heads, head_dim]`` -> rotated copy.  ``positions``
        (``[b, s]`` or ``[b*s]``, any integer dtype): table row per token."""
        b, s, h, d = x.shape
        if d != self.head_dim:
            raise ValueError(f"expected head_dim {self.head_dim}, got {d}")
        if positions is None:
            if b > self.max_seq_len_cached:  # rotary.py:58-59 (its "seq_len" is the batch size)
                self._update_rope_cache(b)
            positions = torch.arange(b, device=x.device, dtype=torch.int32).repeat_interleave(s)
        else:
            positions = positions.reshape(-1).to(device=x.device, dtype=torch.int32)
            if positions.numel() != b * s:
                raise ValueError("one position per token")
        out = x.reshape(b * s, h, d).clone(memory_format=torch.contiguous_format)
        paged_ops.rope_kv_append(out, None, None, None, None, None, positions.contiguous(), self.cos_emb,
                                 self.sin_emb)
        return out.view(b, s, h, d)
