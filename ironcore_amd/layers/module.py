"""Base class of the layers, mirroring what the attention path needs from the
reference's BaseModule (ironcore/layers/module.py:19-41) and its dtype helper
(ironcore/utils.py:129-143)."""
from __future__ import annotations

import math

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

    def init_weights(self):
        """ironcore/layers/module.py:43-76 at tensor-parallel size 1: biases 0,
        norm scales 1, every other parameter N(0, init_std) (Xavier-uniform when
        ``init.xavier_init`` is set), the residual projections then re-drawn
        from N(0, init_std / sqrt(2 * num_layers))."""
        if self.config.trainer.tensor_model_parallel_size != 1:
            raise NotImplementedError("sharded initialisation (tensor_model_parallel_size > 1) is not built: one GPU")
        with torch.no_grad():
            for name, param in self.named_parameters():
                if "bias" in name:
                    param.zero_()
                    continue
                if "norm" in name:
                    param.fill_(1.0)
                    continue
                if self.xavier_init:
                    torch.nn.init.xavier_uniform_(param)
                else:
                    param.normal_(mean=0.0, std=self.init_std)
                if name.endswith("output.weight") or name.endswith("down_proj.weight"):
                    param.normal_(mean=0.0, std=self.init_std / math.sqrt(2 * self.config.model.num_layers))
