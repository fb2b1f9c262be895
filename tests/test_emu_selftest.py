"""The wave64 emulator against the documented semantics of the instructions it models (tests/emu/selftest.cpp): MFMA
operand layouts against a plain matrix product, the lane permutes, the transposing LDS read, and the model of
asynchronous global -> LDS copies (a read that the proper wait does not cover must see stale LDS)."""
import ctypes
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "emu"))


@pytest.fixture(scope="module")
def emu():
    import build_emu
    return ctypes.CDLL(build_emu.build())


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("shape,m,k", [(0, 32, 16), (1, 16, 32), (2, 16, 16)])
def test_mfma_is_a_matrix_product_in_the_documented_layout(emu, shape, m, k):
    g = torch.Generator().manual_seed(shape)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16)
    b = torch.randn(k, m, generator=g).to(torch.bfloat16)
    d = torch.zeros(m, m)
    assert emu.emu_selftest_mfma(shape, _p(a), _p(b), _p(d)) == 0
    assert torch.allclose(d, a.float() @ b.float() + 1.0, atol=1e-5)


def test_lane_permutes(emu):
    out = torch.zeros(194)
    assert emu.emu_selftest_lanes(_p(out)) == 0
    lanes = np.arange(64)
    assert (out[:64].numpy() == (lanes % 32) * 2 + 32).all()                       # lanes l and l ^ 32
    x = lanes * 7 % 64
    want = np.array([max(x[l % 16 + 16 * r] for r in range(4)) for l in lanes])    # the four lanes that share l % 16
    assert (out[64:128].numpy() == want).all()
    assert (out[128:192].numpy() == (63 - lanes % 4) * 3).all()
    mask = sum(1 << l for l in range(64) if l % 3 == 0)
    assert int(out[192]) == mask & 0xffff and int(out[193]) == mask >> 48


def test_transposing_lds_read(emu):
    out = torch.zeros(256, dtype=torch.int16)
    assert emu.emu_selftest_transpose(_p(out)) == 0
    got = out.view(64, 4).numpy()
    for l in range(64):
        g, i = divmod(l, 16)
        assert list(got[l]) == [(4 * g + k) * 16 + i for k in range(4)]           # column i of rows 4g .. 4g+3


def test_a_read_without_the_wait_sees_stale_lds(emu):
    if not emu.emu_selftest_late_loads():
        pytest.skip("EMU_LATE_LOADS=0: copies land at once")
    src = torch.arange(512, dtype=torch.int32) + 1000
    stale = 0xFFFFFFFF - (1 << 32)                                                  # LDS is poisoned with 0xff before every workgroup
    out = torch.zeros(512, dtype=torch.int32)
    assert emu.emu_selftest_async(0, _p(src), _p(out)) == 0
    assert torch.equal(out, src)                                                    # waited for everything
    assert emu.emu_selftest_async(1, _p(src), _p(out)) == 0
    assert torch.equal(out[:256], src[:256]) and (out[256:] == stale).all()         # the newest request may still be in flight
    assert emu.emu_selftest_async(2, _p(src), _p(out)) == 0
    assert (out == stale).all()


_RACE = """
import ctypes, sys, torch
emu = ctypes.CDLL(sys.argv[1])
out = torch.zeros(2, dtype=torch.int32)
assert emu.emu_selftest_race(ctypes.c_void_p(out.data_ptr())) == 0
print(out[0].item(), out[1].item())
"""


@pytest.mark.parametrize("order", ["forward", "reverse"])
def test_the_wave_that_runs_first_sees_a_missing_barrier(order):
    """Waves run first to last between barriers, last to first with EMU_ORDER=reverse: of two waves that read each other's
    LDS word without a barrier, the one that runs first reads the poison (-1), the other one the value (wave number + 1).
    A kernel that passes under both orders has no such read in either direction."""
    import subprocess
    import build_emu
    env = dict(os.environ, EMU_ORDER=order)
    r = subprocess.run([sys.executable, "-c", _RACE, build_emu.build()], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert r.stdout.split() == (["-1", "1"] if order == "forward" else ["2", "-1"]), r.stdout


def test_an_instruction_no_lane_takes_part_in_is_an_error(emu):
    """The waits count global -> LDS instructions per wave, and one that every lane is masked off for is never issued:
    a kernel that masks lanes (padded head dims) must keep a lane on each.  One real lane is enough; none fails the launch."""
    src = torch.arange(256, dtype=torch.int32)
    assert emu.emu_selftest_masked(_p(src), 64) == 0
    assert emu.emu_selftest_masked(_p(src), 1) == 0
    assert emu.emu_selftest_masked(_p(src), 0) != 0
