"""flash_ck.ops.fmha: the functional FMHA API (the reference declares this family and leaves it empty,
flash_ck/utils/utils.py:49-58).  The operators live in flashck_amd.ops.fmha; this is their name in the reference's layout."""
from flashck_amd.ops.fmha import *  # noqa: F401,F403
from flashck_amd.ops.fmha import __all__  # noqa: F401
