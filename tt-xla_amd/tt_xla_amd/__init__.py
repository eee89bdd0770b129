"""MI355X-native paged KV-cache write and paged attention behind tt-xla's operator
and attention-backend interface.

Importing the package registers the ``torch.ops.tt.*`` operators for HIP devices
(``custom_ops``); ``attention`` and ``attention_mla`` hold the vLLM-facing backend classes and ``metadata``
the host-side construction of their per-pass page tables and positions.  Every operator
runs a hand-written gfx950 kernel from ``lib/libttpa.so``; there is no other
implementation to fall back to, and a missing library is an error.
"""

from . import _native  # noqa: F401
from . import custom_ops  # noqa: F401
from .attention import TTAttentionBackend, TTAttentionBackendImpl, TTMetadata  # noqa: F401
from .attention_mla import TTMLAAttentionBackend, TTMLAAttentionBackendImpl  # noqa: F401
from .metadata import PagedMetadataBuilder  # noqa: F401

__all__ = ["TTAttentionBackend", "TTAttentionBackendImpl", "TTMLAAttentionBackend",
           "TTMLAAttentionBackendImpl", "TTMetadata", "PagedMetadataBuilder", "custom_ops"]
