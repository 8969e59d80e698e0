"""Public operation API, importable the way ``ejkernel.modules`` is
(ejkernel/modules/__init__.py:68-70,88-89)."""

from .operations import (
    BaseOperationConfig,
    RaggedPageAttention,
    RaggedPageAttentionConfig,
    RaggedPageAttentionv3,
    RaggedPageAttentionv3Config,
    ragged_page_attention,
    ragged_page_attention_v3,
)

__all__ = ["BaseOperationConfig", "RaggedPageAttention", "RaggedPageAttentionConfig", "RaggedPageAttentionv3",
           "RaggedPageAttentionv3Config", "ragged_page_attention", "ragged_page_attention_v3"]
