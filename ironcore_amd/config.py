"""The slice of the reference's configuration that the attention path reads.

The reference threads one ``MainConfig`` through every module constructor
(ironcore/config/__init__.py:33-44).  The attention layer and the modules on
either side of it read only a handful of fields; this module declares exactly
those, with the reference's names and defaults, so that the same constructor
call ``Attention(config)`` works with either this object or the reference's
own ``MainConfig`` (attribute access is all that is used).

  model.*      ironcore/config/config_model.py:39-154
  trainer.*    ironcore/config/config_trainer.py:79-99
  init.*       ironcore/config/config_trainer.py:164-176
  operation.*  ironcore/config/config_trainer.py:137-148
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass
class PositionalEmbeddingConfig:
    type: str = "absolute"
    base: int = 10000
    scaling_factor: float = 1.0
    offset: int = 0


@dataclass
class ModelConfig:
    d_model: int = 512
    d_ffn: int = 2048
    num_layers: int = 2
    num_attention_heads: int = 8
    num_attention_groups: Optional[int] = None
    head_dim: int = 128
    max_seq_len: int = 512
    max_position_embeddings: int = 512
    dropout_embd: float = 0.1
    dropout_attn: float = 0.1
    dropout_mlp: float = 0.1
    precision: str = "bfloat16"
    untie_embed: bool = False
    no_bias: bool = False
    ln_type: str = "layernorm"
    ln_eps: float = 1e-5
    post_ln: bool = False
    activation_type: str = "gelu"
    fp32_residual_connection: bool = False
    positional_embedding: PositionalEmbeddingConfig = field(default_factory=PositionalEmbeddingConfig)

    def __post_init__(self):
        if self.ln_type not in ("layernorm", "rmsnorm"):
            raise ValueError(f"Invalid layer norm type: {self.ln_type}")
        if self.num_attention_groups is None:
            self.num_attention_groups = self.num_attention_heads


@dataclass
class TrainerConfig:
    tensor_model_parallel_size: int = 1
    use_flash_attn: bool = True
    vocab_padding_unit: int = 128


@dataclass
class InitConfig:
    seed: int = 42
    init_std: float = 0.006
    xavier_init: Optional[bool] = False


@dataclass
class OperationConfig:
    activation_recompute: bool = False
    recompute_strategy: Optional[str] = None


@dataclass
class MainConfig:
    model: ModelConfig = field(default_factory=ModelConfig)
    trainer: TrainerConfig = field(default_factory=TrainerConfig)
    init: InitConfig = field(default_factory=InitConfig)
    operation: OperationConfig = field(default_factory=OperationConfig)


def gpt2_small_config(precision: str = "fp32") -> MainConfig:
    """GPT-2 small dimensions (reference: configs/model/gpt2-small.yaml:1-9):
    12 layers, 12 heads, head_dim 64, d_model 768, d_ffn 3072, learned absolute
    positions, LayerNorm with bias, exact GELU, tied embeddings, no dropout at
    inference."""
    return MainConfig(
        model=ModelConfig(d_model=768, d_ffn=3072, num_layers=12, num_attention_heads=12,
                          num_attention_groups=12, head_dim=64, max_seq_len=1024,
                          max_position_embeddings=1024, dropout_embd=0.0, dropout_attn=0.0,
                          dropout_mlp=0.0, precision=precision),
        trainer=TrainerConfig(use_flash_attn=False),
        init=InitConfig(seed=0, init_std=0.02))
