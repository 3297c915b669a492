from .attention import Attention, PagedAttentionMetadata
from .module import BaseModule, get_model_dtype
from .rotary import RotaryPositionalEmbedding

__all__ = ["Attention", "PagedAttentionMetadata", "BaseModule", "get_model_dtype", "RotaryPositionalEmbedding"]
