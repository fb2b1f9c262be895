from .fmha import *  # noqa: F401,F403
from .fmha import __all__  # noqa: F401
