"""Drop-in for the reference's ``streaming_attention`` package
(src/streaming_attention/__init__.py:1): same two public names."""
from .api import streaming_attention, streaming_attention_reference

__all__ = ["streaming_attention", "streaming_attention_reference"]
