"""Operation registry with the surface of FlashCK's flash_ck/utils/utils.py:21-130.

There the FMHA slot is declared but never filled (flash_ck/utils/utils.py:49-58); here it is the one that is
registered, by flashck_amd.ops.fmha at import time.
"""
from enum import Enum
from typing import Callable, Dict, Optional

__all__ = ["FlashCKOperationType", "is_available", "get_flashck_functions", "register_flashck_functions",
           "get_available_operations", "get_operation_function"]


class FlashCKOperationType(Enum):
    LAYER_NORM = "layer_norm"
    FMHA = "fmha"
    GEMM = "gemm"


_FLASHCK_FUNCTIONS: Dict[str, Dict[str, Callable]] = {}
_FLASHCK_AVAILABILITY: Dict[str, bool] = {t.value: False for t in FlashCKOperationType}


def is_available(operation_type: Optional[str] = None) -> bool:
    if operation_type is None:
        return any(_FLASHCK_AVAILABILITY.values())
    return _FLASHCK_AVAILABILITY.get(operation_type, False)


def get_flashck_functions(operation_type: str) -> Optional[Dict[str, Callable]]:
    if not is_available(operation_type):
        return None
    return _FLASHCK_FUNCTIONS.get(operation_type)


def register_flashck_functions(operation_type: str, functions: Dict[str, Callable]) -> None:
    _FLASHCK_FUNCTIONS[operation_type] = dict(functions)
    _FLASHCK_AVAILABILITY[operation_type] = True


def get_available_operations() -> Dict[str, bool]:
    return _FLASHCK_AVAILABILITY.copy()


def get_operation_function(operation_type: str, function_name: str) -> Optional[Callable]:
    fns = get_flashck_functions(operation_type)
    return None if fns is None else fns.get(function_name)
