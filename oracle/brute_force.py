"""Float64 loop form of masked softmax attention (TEST INFRASTRUCTURE).

Written from the mathematical definition, with no tensor library calls in the
arithmetic, so that an indexing or ordering mistake in the torch restatement
(a transposed operand, a wrong GQA head map, a mask applied to the wrong
axis, scale on the wrong side) shows up as a mismatch on tiny shapes.
"""
from __future__ import annotations

import math

import numpy as np


def attention_f64(q: np.ndarray, k: np.ndarray, v: np.ndarray,
                  mask: np.ndarray | None = None) -> np.ndarray:
    """q [b,sq,hn,hd], k/v [b,sk,gn,hd], mask [b or 1, sq, sk] (nonzero =
    visible) or None.  Returns [b, sq, hn*hd] float64 with channel index
    h*hd + d."""
    b, sq, hn, hd = q.shape
    sk, gn = k.shape[1], k.shape[2]
    group = hn // gn
    out = np.zeros((b, sq, hn * hd), dtype=np.float64)
    for bi in range(b):
        for h in range(hn):
            g = h // group
            for i in range(sq):
                logits = []
                for j in range(sk):
                    if mask is not None and not mask[bi if mask.shape[0] > 1 else 0, i, j]:
                        logits.append(-math.inf)
                        continue
                    dot = 0.0
                    for d in range(hd):
                        dot += float(q[bi, i, h, d]) * float(k[bi, j, g, d])
                    logits.append(dot / math.sqrt(hd))
                top = max(logits)
                weights = [math.exp(x - top) if x != -math.inf else 0.0 for x in logits]
                total = sum(weights)
                for d in range(hd):
                    acc = 0.0
                    for j in range(sk):
                        acc += weights[j] * float(v[bi, j, g, d])
                    out[bi, i, h * hd + d] = acc / total
    return out
