"""Public operation API, importable the way ``ejkernel.modules`` is
(ejkernel/modules/__init__.py:68-69,88)."""

from .operations import BaseOperationConfig, RaggedPageAttention, RaggedPageAttentionConfig, ragged_page_attention

__all__ = ["BaseOperationConfig", "RaggedPageAttention", "RaggedPageAttentionConfig", "ragged_page_attention"]
