"""MI355X-native FMHA forward path with FlashCK's operator surface (one GPU, gfx950).

Importing the package never touches the GPU; `flashck_amd.ops.fmha` loads the HIP library on first use and
raises if it has not been built (`python -m flashck_amd.build`).
"""
from .utils import (get_flag_value, print_all_flags, print_flag_info, set_flag_value,  # noqa: F401
                    FlashCKOperationType, get_available_operations, get_flashck_functions,  # noqa: F401
                    get_operation_function, is_available, register_flashck_functions)
from . import ops  # noqa: F401
from . import nn  # noqa: F401

__version__ = "0.1.0"
