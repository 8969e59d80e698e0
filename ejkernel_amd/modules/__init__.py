"""Public operation API, importable the way ``ejkernel.modules`` is
(ejkernel/modules/__init__.py:68-70,88-89)."""

from .operations import (
    BaseOperationConfig,
    FwdParams,
    PageAttention,
    PageAttentionConfig,
    RaggedDecodeAttention,
    RaggedDecodeAttentionConfig,
    RaggedPageAttention,
    RaggedPageAttentionConfig,
    RaggedPageAttentionv3,
    RaggedPageAttentionv3Config,
    page_attention,
    ragged_decode_attention,
    ragged_page_attention,
    ragged_page_attention_v3,
)

__all__ = ['BaseOperationConfig', 'FwdParams', 'PageAttention', 'PageAttentionConfig', 'RaggedDecodeAttention', 'RaggedDecodeAttentionConfig', 'RaggedPageAttention', 'RaggedPageAttentionConfig', 'RaggedPageAttentionv3', 'RaggedPageAttentionv3Config', 'page_attention', 'ragged_decode_attention', 'ragged_page_attention', 'ragged_page_attention_v3']
