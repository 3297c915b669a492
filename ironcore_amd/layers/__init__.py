from .attention import Attention, PagedAttentionMetadata
from .module import BaseModule, get_model_dtype

__all__ = ["Attention", "PagedAttentionMetadata", "BaseModule", "get_model_dtype"]
