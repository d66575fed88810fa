"""Drop-in for the reference's ``streaming_attention`` package
(src/streaming_attention/__init__.py:1): same two public names, plus ``compiled_wrapper`` to choose
the reference's ``torch.compile`` call path per call site."""
from .api import compiled_wrapper, streaming_attention, streaming_attention_reference

__all__ = ["streaming_attention", "streaming_attention_reference", "compiled_wrapper"]
