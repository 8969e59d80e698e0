from .configs import BaseOperationConfig, PageAttentionConfig, RaggedPageAttentionConfig, RaggedPageAttentionv3Config
from .page_attention import PageAttention, page_attention
from .ragged_page_attention import RaggedPageAttention, ragged_page_attention
from .ragged_page_attention_v3 import RaggedPageAttentionv3, ragged_page_attention_v3

__all__ = ["BaseOperationConfig", "PageAttention", "PageAttentionConfig", "RaggedPageAttention",
           "RaggedPageAttentionConfig", "RaggedPageAttentionv3", "RaggedPageAttentionv3Config", "page_attention",
           "ragged_page_attention", "ragged_page_attention_v3"]
