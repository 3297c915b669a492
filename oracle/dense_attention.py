"""Dense attention oracle (TEST INFRASTRUCTURE, not product code).

Restates the arithmetic of the reference's dense attention method
(ironcore/layers/attention.py:68-142) as one free function.  The op sequence
and the dtype of every intermediate match the reference so that, in bf16, the
same values are rounded at the same places:

    q [b,sq,hn,hd] -> [b,hn,sq,hd]            attention.py:89
    k [b,sk,gn,hd] -> [b,gn,hd,sk]            attention.py:90
    v [b,sk,gn,hd] -> [b,gn,sk,hd]            attention.py:91
    GQA: K and V heads repeated hn//gn times, so query head h reads
         KV head h // (hn//gn)                attention.py:95-102
    scores = q @ k                            attention.py:107
    scores = scores / sqrt(hd)                attention.py:110  (after the matmul)
    scores[mask == 0] = finfo(dtype).min      attention.py:115-117
    scores -= rowmax(scores)                  attention.py:121-122
    probs = softmax(scores, -1)               attention.py:124
    out = probs @ v                           attention.py:134
    out -> [b, sq, hn*hd] (head-major)        attention.py:137-140

Dropout (attention.py:128-129) is the identity at inference and is left out.
"""
from __future__ import annotations

import torch


def mask_fill_value(dtype: torch.dtype) -> float:
    """Value written where the mask hides a key: the most negative finite
    number of the model dtype, not -inf (attention.py:66)."""
    return torch.finfo(dtype).min


def dense_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                    attention_mask: torch.Tensor | None = None) -> torch.Tensor:
    """query [b,sq,hn,hd], key/value [b,sk,gn,hd], mask broadcastable to
    [b,1,sq,sk] with nonzero = visible.  Returns [b, sq, hn*hd] in the input
    dtype."""
    b, sq, hn, hd = query.shape
    sk, gn = key.shape[1], key.shape[2]
    if hn % gn != 0:
        raise ValueError("query heads must be a multiple of KV heads")
    rep = hn // gn

    qh = query.transpose(1, 2)
    kh = key.permute(0, 2, 3, 1)
    vh = value.transpose(1, 2)
    if rep != 1:
        kh = kh.repeat_interleave(rep, dim=1)
        vh = vh.repeat_interleave(rep, dim=1)

    scores = torch.matmul(qh, kh)
    scores = scores / (hd ** 0.5)
    scores = scores.view(b, hn, sq, sk)
    if attention_mask is not None:
        scores = scores.masked_fill(attention_mask == 0, mask_fill_value(query.dtype))

    scores = scores - scores.max(dim=-1, keepdim=True)[0]
    probs = torch.softmax(scores, dim=-1)

    ctx = torch.matmul(probs, vh)
    return ctx.transpose(1, 2).reshape(b, sq, -1)


def causal_offset_mask(sq: int, sk: int, device=None) -> torch.Tensor:
    """Mask for a query chunk of length sq that follows sk - sq cached tokens:
    mask[i, j] = (j <= (sk - sq) + i), shape [1,1,sq,sk], bool.  With sq == sk
    this is the lower-triangular mask the reference model builds
    (ironcore/language_model.py:109-114,159)."""
    prefix = sk - sq
    i = torch.arange(sq, device=device).unsqueeze(1)
    j = torch.arange(sk, device=device).unsqueeze(0)
    return (j <= prefix + i).view(1, 1, sq, sk)
