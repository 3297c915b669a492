"""Base class of the layers, mirroring what the attention path needs from the
reference's BaseModule (ironcore/layers/module.py:19-41) and its dtype helper
(ironcore/utils.py:129-143)."""
from __future__ import annotations

import torch


def get_model_dtype(config) -> torch.dtype:
    """Model dtype named by ``config.model.precision`` (ironcore/utils.py:129-143)."""
    name = config.model.precision.lower()
    if name in ("bfloat16", "bf16"):
        return torch.bfloat16
    if name in ("float16", "fp16"):
        return torch.float16
    return torch.float


class BaseModule(torch.nn.Module):
    """Keeps the config and the init/recompute fields every reference module
    reads in its constructor (ironcore/layers/module.py:24-34)."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.init_std = config.init.init_std
        self.xavier_init = config.init.xavier_init
        self.use_reentrant = config.operation.recompute_strategy == "optimized"
