"""Runtime flags: the `get_flag_value` / `set_flag_value` / `print_all_flags` / `print_flag_info` surface of the
reference's Python module (core/pybind/pybind.cc:21-44), with the flags of core/utils/flags.cc:153-239 that mean
something for a prebuilt kernel library (the tuning group).  Values travel as strings, as they do there; a flag takes its
initial value from the environment variable of the same name.
"""
import os
from typing import Dict, NamedTuple, Union

__all__ = ["get_flag_value", "set_flag_value", "print_all_flags", "print_flag_info", "get_all_flag_info", "flag"]


class FlagInfo(NamedTuple):
    name: str
    type: type
    default: Union[bool, int, str]
    doc: str
    is_writable: bool


_TRUE, _FALSE = ("1", "true", "t", "yes", "y", "on"), ("0", "false", "f", "no", "n", "off")


def _parse(info: FlagInfo, text: str):
    if info.type is bool:
        low = text.strip().lower()
        if low in _TRUE:
            return True
        if low in _FALSE:
            return False
        raise ValueError(f"not a boolean: {text!r}")
    if info.type is int:
        v = int(text.strip(), 0)
        if not -2 ** 31 <= v < 2 ** 31:
            raise ValueError(f"out of int32 range: {text!r}")
        return v
    return text


def _format(value) -> str:
    if isinstance(value, bool):
        return "true" if value else "false"
    return str(value)


_REGISTRY: Dict[str, FlagInfo] = {}
_VALUES: Dict[str, Union[bool, int, str]] = {}


def _define(name, default, doc, writable=True):
    info = FlagInfo(name, type(default), default, doc, writable)
    _REGISTRY[name] = info
    value = default
    env = os.environ.get(name)
    if env is not None:
        try:
            value = _parse(info, env)
        except ValueError as e:
            raise ValueError(f"environment variable {name}: {e}") from None
    _VALUES[name] = value


# names, defaults and help texts follow core/utils/flags.cc:157,201-233 unless noted
# here: every paged launch of the Python operators is preceded by a device-side check of its block table / page list
_define("FC_DEBUG_KERNEL_INSTANCE", False, "Enable kernel instance debugging")
_define("FC_TUNING_DB_DIR", "", "Directory for profiler cache storage")
_define("FC_FORCE_PROFILING", False, "Force profiling even if cached results exist")  # reference default: true
_define("FC_FLUSH_PROFILING_DB", False, "Flush profile cache database on startup")
# reference default is 1; a prebuilt library has nothing to tune unless asked, so cached choices are used when there are any
_define("FC_TUNING_MODE", 2, "Tuning mode: 0=heuristic, 1=autotuning, 2=hybrid")
_define("FC_TUNING_METRIC", 0, "Profiling metric: 0=latency, 1=throughput(TFLOPS), 2=bandwidth")
_define("FC_TUNING_NUM_COLD_ITERATION", 16, "Number of warm-up iterations for profiling")
_define("FC_TUNING_NUM_REPEATS", 64, "Number of profiling iterations for measurements")
_define("FC_TUNING_GPU_TIMER", True, "Enable GPU timer for accurate profiling", writable=False)
_define("FC_TUNING_SEED", 42, "Random seed for tuning")
_define("FC_TUNING_LOG", False, "Enable detailed tuning logs")
_define("FC_TUNING_FLUSH_CACHE", True, "Flush cache before profiling measurements")
_define("FC_TUNING_ROTATING_COUNT", 1, "Number of rotating profiling runs")


def get_flag_value(name: str) -> str:
    """Current value as a string; RuntimeError('Flag not found: <name>') for an unknown flag."""
    if name not in _REGISTRY:
        raise RuntimeError("Flag not found: " + name)
    return _format(_VALUES[name])


def set_flag_value(name: str, value: str) -> None:
    """Set a flag from a string; RuntimeError('Failed to set flag: <name>') when the flag is unknown, read-only or
    the text does not parse as the flag's type."""
    info = _REGISTRY.get(name)
    if info is None or not info.is_writable:
        raise RuntimeError("Failed to set flag: " + name)
    try:
        _VALUES[name] = _parse(info, _format(value))
    except ValueError:
        raise RuntimeError("Failed to set flag: " + name) from None


def flag(name: str):
    """Typed value, for use inside the package."""
    return _VALUES[name]


def get_all_flag_info(writable_only: bool = False) -> Dict[str, FlagInfo]:
    return {n: i for n, i in sorted(_REGISTRY.items()) if i.is_writable or not writable_only}


_TYPE_NAME = {bool: "bool", int: "int32_t", str: "string"}


def print_all_flags(writable_only: bool = False) -> None:
    print("\n=== FlashCK Flags ===")
    print(f"{'Flag Name':<30}{'Current Value':<15}{'Default Value':<15}{'Writable':<8}Description")
    print("-" * 80)
    for name, info in get_all_flag_info(writable_only).items():
        print(f"{name:<30}{get_flag_value(name):<15}{_format(info.default):<15}{'Yes' if info.is_writable else 'No':<8}{info.doc}")
    print()


def print_flag_info(name: str) -> None:
    info = _REGISTRY.get(name)
    if info is None:
        print(f"Flag '{name}' not found.")
        raise RuntimeError("Flag not found: " + name)
    print("\n=== Flag Information ===")
    print(f"Name: {info.name}")
    print(f"Current Value: {get_flag_value(name)}")
    print(f"Default Value: {_format(info.default)}")
    print(f"Type: {_TYPE_NAME[info.type]}")
    print(f"Writable: {'Yes' if info.is_writable else 'No'}")
    print(f"Description: {info.doc}\n")
