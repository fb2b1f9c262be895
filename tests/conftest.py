import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """tests/test_emu_kernels.py re-runs the GPU test functions on the CPU emulator; by default only the cases named in
    tests/emu/quick_cases.txt (about two minutes in one process), all of them with FCK_EMU_FULL=1."""
    if os.environ.get("FCK_EMU_FULL") == "1":
        return
    try:
        with open(os.path.join(ROOT, "tests", "emu", "quick_cases.txt")) as f:
            quick = {line.strip() for line in f if line.strip() and not line.startswith("#")}
    except OSError:
        quick = set()
    for item in items:
        if item.module.__name__ == "test_emu_kernels" and item.name not in quick:
            item.add_marker(pytest.mark.skip(reason="not in the emulator's quick set; FCK_EMU_FULL=1 runs it"))


@pytest.fixture(scope="session")
def orc():
    from oracle import fmha_oracle
    fmha_oracle.build()
    return fmha_oracle


@pytest.fixture(scope="session")
def fmha():
    """The HIP operators; a GPU test that gets here without the built library must fail, not skip."""
    import torch
    from flashck_amd import _lib
    from flashck_amd.ops import fmha as ops
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    _lib.load()
    # the library under test is the in-tree build, never another copy
    want = os.path.join(ROOT, "flashck_amd", "libflashck_fmha.so")
    assert os.path.realpath(_lib.LIB_PATH) == os.path.realpath(want), f"tests loaded {_lib.LIB_PATH}, not {want}"
    return ops
