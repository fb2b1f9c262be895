"""Module wrappers, as in the reference's flash_ck/nn."""
from flashck_amd.nn import Attention, PagedAttention  # noqa: F401

__all__ = ["Attention", "PagedAttention"]
