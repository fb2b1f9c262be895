"""Functional operators by family, as in the reference's flash_ck/ops."""
from . import fmha  # noqa: F401
