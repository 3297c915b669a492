"""Multiple-choice scoring on the prefill kernel: the arithmetic of the
reference's HellaSwag task (ironcore/eval/tasks/hellaswag.py:63-88 and
:144-175) without its dataset and tokenizer plumbing.

A batch of token sequences ``[b, s]`` (one per (prompt, ending) pair, padded
to a common length) goes through one causal pass of the model, sq = sk with no
cached prefix, which is the chunked-prefill MFMA kernel at prefix 0; the score
of a sequence is the mean cross-entropy of its next-token predictions.
"""
from __future__ import annotations

from typing import Sequence

import torch
import torch.nn.functional as F


@torch.no_grad()
def per_sample_losses(model, tokenized_inputs: torch.Tensor) -> torch.Tensor:
    """hellaswag.py:63-88: inputs are ``tokenized_inputs[:, :-1]``, labels
    ``tokenized_inputs[:, 1:]``; returns the mean cross-entropy per sequence
    (over every position, padding included, exactly as the reference does),
    fp32 on the CPU."""
    input_ids = tokenized_inputs[:, :-1]
    labels = tokenized_inputs[:, 1:]
    logits = model(input_ids)  # [b, s, v]
    losses = [F.cross_entropy(logits[i].float(), labels[i], reduction="mean") for i in range(logits.size(0))]
    return torch.stack(losses).cpu()


def pick_endings(prompts: Sequence, losses: Sequence[float], labels: Sequence[int]) -> dict:
    """hellaswag.py:144-175: consecutive entries with the same prompt form one
    question; the ending with the lowest loss is the prediction, correct when
    its label is 1.  Returns ``{"metric": "accuracy", "score": percent}``."""
    if len(prompts) == 0:
        return 0.0
    total_score = total_samples = 0
    i = 0
    while i < len(losses):
        current = prompts[i]
        cur_losses, cur_labels = [], []
        while i < len(prompts) and prompts[i] == current:
            cur_losses.append(float(losses[i]))
            cur_labels.append(int(labels[i]))
            i += 1
        total_score += cur_losses.index(min(cur_losses)) == cur_labels.index(1)
        total_samples += 1
    return {"metric": "accuracy", "score": total_score / total_samples * 100}
