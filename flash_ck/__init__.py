"""flash_ck: the package and module names of the reference (flash_ck/__init__.py, core/pybind/pybind.cc:13-58), with the
FMHA forward family behind them.

    flash_ck.fmha_fwd(...), flash_ck.fmha_fwd_splitkv(...), ...   compiled functions of torch tensors (flash_ck.flash_ck)
    flash_ck.ops.fmha.*                                           functional API with validation, workspaces, tuning
    flash_ck.nn.Attention / PagedAttention                        module wrappers
    flash_ck.get_flag_value / set_flag_value / ...                runtime flags
    flash_ck.is_available / get_available_operations              operation registry

Both the compiled functions and the functional API end in the C ABI of libflashck_fmha.so (the gfx950 kernels); when
that library or the compiled module has not been built, importing this package fails with the build command."""
import os as _os

try:
    from .flash_ck import (fmha_batch_prefill, fmha_fwd, fmha_fwd_appendkv, fmha_fwd_pagedkv, fmha_fwd_splitkv,  # noqa: F401
                           fmha_fwd_splitkv_combine, fmha_fwd_varlen, fmha_last_kernel, fmha_num_splits_heuristic, fmha_version)
except ImportError as e:  # no fallback: say how to build
    raise ImportError(f"the compiled module flash_ck.flash_ck is missing or does not load ({e}); build it with "
                      f"`python -m flash_ck.build` in {_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__)))}") from e

from . import nn, ops  # noqa: E402,F401
from .nn import Attention, PagedAttention  # noqa: E402,F401
from .utils import (get_available_operations, get_flag_value, is_available, print_all_flags, print_flag_info,  # noqa: E402,F401
                    set_flag_value)

__version__ = "0.2.0"

__all__ = ["ops", "nn", "fmha_fwd", "fmha_fwd_varlen", "fmha_fwd_splitkv", "fmha_fwd_splitkv_combine", "fmha_fwd_appendkv",
           "fmha_batch_prefill", "fmha_fwd_pagedkv", "fmha_num_splits_heuristic", "fmha_version", "fmha_last_kernel", "Attention",
           "PagedAttention", "is_available", "get_available_operations", "get_flag_value", "set_flag_value", "print_all_flags",
           "print_flag_info"]
