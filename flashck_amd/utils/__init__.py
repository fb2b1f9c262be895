from .registry import (FlashCKOperationType, get_available_operations, get_flashck_functions,  # noqa: F401
                       get_operation_function, is_available, register_flashck_functions)
from . import flags, tuning  # noqa: F401
from .flags import get_flag_value, print_all_flags, print_flag_info, set_flag_value  # noqa: F401
