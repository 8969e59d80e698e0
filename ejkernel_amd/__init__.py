"""MI355X-native ragged paged attention forward behind ejkernel's call signature.

``from ejkernel_amd.modules import ragged_page_attention, RaggedPageAttention,
RaggedPageAttentionConfig`` mirrors ``from ejkernel.modules import ...``
(ejkernel/modules/__init__.py:68-69,88).  There is one implementation: hand-written
HIP kernels for gfx950 in ``librpa_mi355x.so`` reached through a C ABI.
"""

__version__ = "0.1.0"
