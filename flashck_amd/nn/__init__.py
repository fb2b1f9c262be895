"""Module wrappers over the functional FMHA operators (the `flash_ck.nn` surface of the reference)."""
from .attention import Attention, PagedAttention  # noqa: F401

__all__ = ["Attention", "PagedAttention"]
