"""Registry and flags under the reference's names (flash_ck/utils/utils.py:77-135, core/pybind/pybind.cc:21-44)."""
from flashck_amd.utils import (FlashCKOperationType, get_available_operations, get_flashck_functions, get_flag_value,  # noqa: F401
                               is_available, print_all_flags, print_flag_info, register_flashck_functions, set_flag_value)
