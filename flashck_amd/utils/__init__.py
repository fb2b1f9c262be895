from .registry import (FlashCKOperationType, get_available_operations, get_flashck_functions,  # noqa: F401
                       get_operation_function, is_available, register_flashck_functions)
