"""The kernel sources on a wave64 emulator, on the CPU: the GPU parity tests, re-run without a GPU.

tests/emu/ compiles the UNCHANGED kernel sources of flashck_amd/csrc (and the C ABI in front of them) as host C++ on top
of an emulator that runs every thread of a workgroup as a fiber and makes every cross-lane instruction (MFMA, lane
permutes, readlane, ballot, transposing LDS read) and every barrier a rendezvous.  This module takes the test functions
of the GPU test modules as they are and runs them against that build, with CPU tensors: the same inputs, the same
oracle, the same tolerances.  It shows the kernels' indexing, swizzles, masks, table lookups and arithmetic to be
right; it cannot show timing-dependent faults (a missing wait on an asynchronous load, a race between waves) and it
says nothing about speed.  The emulator is test infrastructure: nothing outside tests/ loads it, and the operators
still refuse to run without the HIP library.

By default only the cases listed in tests/emu/quick_cases.txt run (about two minutes in one process); FCK_EMU_FULL=1
runs every collected case (`FCK_EMU_FULL=1 python -m pytest tests/test_emu_kernels.py -n 8`: several minutes on 8 cores).
Tests that need a real device (graph capture, the C++ header program, timing) are left out by name.
"""
import ctypes
import importlib
import os
import sys

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "emu"))

GPU_MODULES = ["test_gpu_decode", "test_gpu_combine", "test_gpu_appendkv", "test_gpu_prefill", "test_gpu_prefill_grid",
               "test_gpu_score_mods", "test_gpu_head_dims", "test_gpu_step", "test_zr_random_shapes", "test_zs_every_instantiation", "test_zt_prefill_variants", "test_zu_fast_kernel_mods", "test_zv_fp8_cache", "test_zw_validate", "test_zx_fp8_roles", "test_zy_flash_ck_module",
               "test_zz_no_alloc"]
# need a real device: HIP graph capture
NEEDS_DEVICE = {"test_decode_captured_in_a_graph"}

_mods = [importlib.import_module(m) for m in GPU_MODULES]
for _m in _mods:
    for _name in dir(_m):
        _fn = getattr(_m, _name)
        if _name.startswith("test_") and callable(_fn) and _name not in NEEDS_DEVICE:
            globals()[f"test_emu_{_m.__name__[5:]}__{_name[5:]}"] = _fn
del _fn


_PAGE = 4096
_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]


def _guarded_copy(t):
    """A copy of t whose last byte (rounded up to 16) sits right before an inaccessible page: a kernel that reads or
    writes past the end of an input - what ends in a memory access fault on the GPU - takes a segmentation fault here.
    FCK_EMU_GUARD=front puts the page in front of the first byte instead (accesses before the start)."""
    import mmap
    n = t.numel() * t.element_size()
    if n == 0:
        return t.clone()
    n16 = (n + 15) // 16 * 16
    total = (n16 + _PAGE - 1) // _PAGE * _PAGE + _PAGE
    mm = mmap.mmap(-1, total)
    base = ctypes.addressof(ctypes.c_char.from_buffer(mm))
    front = os.environ.get("FCK_EMU_GUARD") == "front"
    guard = base if front else base + total - _PAGE
    if _libc.mprotect(guard, _PAGE, 0) != 0:   # PROT_NONE
        raise OSError(ctypes.get_errno(), "mprotect")
    buf = (ctypes.c_char * n).from_address(base + _PAGE if front else guard - n16)
    buf._mapping = mm   # the tensor keeps buf alive, buf the mapping
    out = torch.frombuffer(buf, dtype=torch.uint8, count=n).view(t.dtype).view(t.shape)
    out.copy_(t.contiguous())
    return out


def _cpu(x, device="cpu"):
    """stand-in for helpers.dev: a private copy on the CPU (kernels write in place, as they do to device copies), placed
    against a guard page"""
    return _guarded_copy(x) if isinstance(x, torch.Tensor) else x


def _wall_timer(fn, cold, repeats):
    """stand-in for tuning.gpu_timer (events on a stream): wall clock around one call; which candidate wins is not
    what these tests check"""
    import time
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


@pytest.fixture(scope="module", autouse=True)
def _emulator_bound():
    """flashck_amd.ops.fmha (and flashck_amd._lib.load) bound to the emulator build for the duration of this module."""
    import build_emu
    import helpers
    from flashck_amd import _lib
    from flashck_amd.ops import fmha as ops
    from flashck_amd.ops.fmha import fmha as F
    from flashck_amd.utils import tuning
    path = build_emu.build()
    lib = ctypes.CDLL(path)
    for name, (res, args) in _lib.SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    saved = dict(lib=_lib._lib, req=F._REQUIRE_GPU_TENSORS, stream=F._stream, sync=torch.cuda.synchronize, device=helpers.DEVICE,
                 timer=tuning.gpu_timer, devs=[(m, m.dev) for m in _mods if hasattr(m, "dev")],
                 streams=[(m, m._stream) for m in _mods if hasattr(m, "_stream")])
    _lib._lib, F._REQUIRE_GPU_TENSORS, F._stream = lib, False, (lambda: None)
    torch.cuda.synchronize = lambda *a, **k: None
    helpers.DEVICE = "cpu"
    tuning.gpu_timer = _wall_timer
    for m, _ in saved["devs"]:
        m.dev = _cpu
    for m, _ in saved["streams"]:
        m._stream = lambda: None
    try:
        yield ops
    finally:
        _lib._lib, F._REQUIRE_GPU_TENSORS, F._stream = saved["lib"], saved["req"], saved["stream"]
        torch.cuda.synchronize = saved["sync"]
        helpers.DEVICE = saved["device"]
        tuning.gpu_timer = saved["timer"]
        for m, d in saved["devs"]:
            m.dev = d
        for m, f in saved["streams"]:
            m._stream = f


@pytest.fixture(scope="module")
def fmha(_emulator_bound):
    return _emulator_bound


@pytest.fixture(scope="module")
def fck(fmha):
    """The glue of the compiled `flash_ck` module (flash_ck/csrc/pybind.cpp), built against the emulator library with
    host tensors allowed, next to the emulator-bound functional API."""
    import types
    import build_emu
    build_emu.build_pybind()
    import flash_ck_emu
    ns = types.SimpleNamespace(**{n: getattr(flash_ck_emu, n) for n in dir(flash_ck_emu) if n.startswith("fmha_")})
    ns.ops = types.SimpleNamespace(fmha=fmha)
    return ns
