from .configs import BaseOperationConfig, RaggedPageAttentionConfig, RaggedPageAttentionv3Config
from .ragged_page_attention import RaggedPageAttention, ragged_page_attention
from .ragged_page_attention_v3 import RaggedPageAttentionv3, ragged_page_attention_v3

__all__ = ["BaseOperationConfig", "RaggedPageAttention", "RaggedPageAttentionConfig", "RaggedPageAttentionv3",
           "RaggedPageAttentionv3Config", "ragged_page_attention", "ragged_page_attention_v3"]
