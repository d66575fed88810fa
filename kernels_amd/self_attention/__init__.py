"""Drop-in for the reference's ``self_attention`` package (src/self_attention/__init__.py):
dense variable-length attention, forward only.  It is the ``context_size >= T`` case of the
streaming forward kernel, so it reuses ``sa_forward`` of libstreaming_attention.so."""
from .kernel import self_attention, self_attention_reference, self_attention_reference_naive

__all__ = ["self_attention", "self_attention_reference", "self_attention_reference_naive"]
