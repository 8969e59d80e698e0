from .configs import (
    BaseOperationConfig,
    FwdParams,
    PageAttentionConfig,
    RaggedDecodeAttentionConfig,
    RaggedPageAttentionConfig,
    RaggedPageAttentionv3Config,
)
from .page_attention import PageAttention, page_attention
from .ragged_decode_attention import RaggedDecodeAttention, ragged_decode_attention
from .ragged_page_attention import RaggedPageAttention, ragged_page_attention
from .ragged_page_attention_v3 import RaggedPageAttentionv3, ragged_page_attention_v3

__all__ = ['BaseOperationConfig', 'FwdParams', 'PageAttention', 'PageAttentionConfig', 'RaggedDecodeAttention', 'RaggedDecodeAttentionConfig', 'RaggedPageAttention', 'RaggedPageAttentionConfig', 'RaggedPageAttentionv3', 'RaggedPageAttentionv3Config', 'page_attention', 'ragged_decode_attention', 'ragged_page_attention', 'ragged_page_attention_v3']
