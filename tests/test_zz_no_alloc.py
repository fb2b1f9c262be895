"""The entry point that allocates nothing (fck_fmha_fwd_splitkv_fused): called through the C ABI, its output must equal
what fck_fmha_fwd_splitkv + fck_fmha_fwd_splitkv_combine give with a caller-owned workspace, on two calls in a row that
share the library's fixed device array, the second with a smaller input."""
import ctypes
import math

import pytest
import torch

from flashck_amd import _lib, generators as gen
import helpers
from helpers import assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu


def _vp(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _run_both(lib, kv, q, ns, mask_type=0, window=(-1, -1), cu=None, max_sq=0):
    """(fused output, two-launch output) through the C ABI; ns > 0 on both paths."""
    B = kv["seqlen_k"].numel()
    Hq, D = q.shape[-2], q.shape[-1]
    Hk, page = kv["k_cache"].shape[2], kv["k_cache"].shape[1]
    sq = q.shape[0] if cu is not None else q.shape[1]
    max_sq = max_sq or sq
    bs = 1 if cu is not None else B
    dt = 4 if q.dtype == torch.bfloat16 else 3
    qd, kc, vc = dev(q), dev(kv["k_cache"]), dev(kv["v_cache"])
    sl, bt, cud = dev(kv["seqlen_k"]), dev(kv["block_table"]), dev(cu)
    scale = 1.0 / math.sqrt(D)
    o_fused = torch.full(q.shape, float("nan"), dtype=q.dtype, device=helpers.DEVICE)
    rc = lib.fck_fmha_fwd_splitkv_fused(_vp(qd), _vp(kc), _vp(vc), None, _vp(o_fused), _vp(cud), None, _vp(sl), _vp(bt), None,
                                        B, sq, 0, Hq, Hk, D, D, max_sq, ns, bt.numel(), page, scale, window[0], window[1],
                                        mask_type, dt, _stream())
    assert rc == 0, lib.fck_last_error().decode()
    o_acc = torch.empty(bs, Hq, ns, sq, D, dtype=torch.float32, device=helpers.DEVICE)
    lse_acc = torch.empty(bs, Hq, ns, sq, dtype=torch.float32, device=helpers.DEVICE)
    o_ref = torch.full(q.shape, float("nan"), dtype=q.dtype, device=helpers.DEVICE)
    rc = lib.fck_fmha_fwd_splitkv(_vp(qd), _vp(kc), _vp(vc), None, _vp(lse_acc), _vp(o_acc), _vp(cud), None, _vp(sl), _vp(bt),
                                  None, B, sq, 0, Hq, Hk, D, D, max_sq, ns, bt.numel(), page, scale, window[0], window[1],
                                  mask_type, dt, _stream())
    assert rc == 0, lib.fck_last_error().decode()
    rc = lib.fck_fmha_fwd_splitkv_combine(_vp(lse_acc), _vp(o_acc), _vp(o_ref), _vp(cud), B, sq, Hq, D, max_sq, ns, dt, _stream())
    assert rc == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    return o_fused, o_ref


def test_fused_equals_two_launches_twice_in_a_row(orc):
    lib = _lib.load()
    g = torch.Generator().manual_seed(77)
    # first call: 14 sequences, 32/8 heads, 5 splits (a grid large enough for the head-pair kernel)
    lens1 = [900, 33, 2048, 1, 517, 1300, 64, 700, 128, 129, 1000, 5, 2500, 333]
    kv1 = gen.paged_kv(lens1, 8, 128, torch.bfloat16, g, 128)
    q1 = gen.randn((len(lens1), 1, 32, 128), torch.bfloat16, g)
    of1, or1 = _run_both(lib, kv1, q1, 5)
    assert_bits_equal(of1, or1, "first call")
    # second call, smaller, right behind the first on the same stream: 2 sequences, 3 splits, ragged queries, causal
    kv2 = gen.paged_kv([130, 700], 2, 128, torch.bfloat16, g, 64)
    cu = torch.tensor([0, 3, 8], dtype=torch.int32)
    q2 = gen.randn((8, 8, 128), torch.bfloat16, g)
    of2, or2 = _run_both(lib, kv2, q2, 3, mask_type=2, window=(-1, 0), cu=cu, max_sq=5)
    assert_bits_equal(of2, or2, "second call")
    # and both agree with the oracle
    ro = orc.fmha_fwd(q1, kv1["k_cache"], kv1["v_cache"], seqlen_k=kv1["seqlen_k"], block_table=kv1["block_table"])
    assert_close(of1, ro, 2e-2, "first call vs oracle")
    ro = orc.fmha_fwd(q2, kv2["k_cache"], kv2["v_cache"], seqstart_q=cu, seqlen_k=kv2["seqlen_k"],
                      block_table=kv2["block_table"], mask_type=2, window=(-1, 0))
    assert_close(of2, ro, 2e-2, "second call vs oracle")


def test_fused_library_chosen_split_count(orc):
    """num_splits = 0: the library's heuristic split count; checked against the oracle."""
    from flashck_amd.ops import fmha
    g = torch.Generator().manual_seed(78)
    for lens, hq, hk in (([3000, 40, 1200, 257, 4096, 1], 32, 8), ([9000, 300], 16, 2)):
        kv = gen.paged_kv(lens, hk, 128, torch.bfloat16, g, 128)
        q = gen.randn((len(lens), 1, hq, 128), torch.bfloat16, g)
        o = fmha.fmha_fwd_splitkv_fused(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), 0, seqlen_k=dev(kv["seqlen_k"]),
                                        block_table=dev(kv["block_table"]))
        ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"])
        assert_close(o, ro, 2e-2, f"auto ranges {lens}")


def test_fused_rejects_what_does_not_fit():
    lib = _lib.load()
    x = torch.zeros(64, dtype=torch.bfloat16, device=helpers.DEVICE)
    i = torch.zeros(64, dtype=torch.int32, device=helpers.DEVICE)
    # 64 sequences x 64 heads x 128 splits x 129 floats > 4 Mi floats
    rc = lib.fck_fmha_fwd_splitkv_fused(_vp(x), _vp(x), _vp(x), None, _vp(x), None, None, _vp(i), _vp(i), None, 64, 1, 0, 64, 8,
                                        128, 128, 1, 128, 64 * 4, 128, 0.1, -1, -1, 0, 4, _stream())
    assert rc == -2 and b"at most" in lib.fck_last_error()


def _other_streams(n):
    """n stream handles besides the current one, and whatever keeps them alive: torch streams on a GPU; under the CPU
    emulator (which runs every launch at once and never looks at the handle) distinct made-up handles."""
    if helpers.DEVICE == "cpu":
        return [ctypes.c_void_p(0x1000 * (i + 1)) for i in range(n)], None
    streams = [torch.cuda.Stream() for _ in range(n)]
    return [ctypes.c_void_p(s.cuda_stream) for s in streams], streams


def test_fused_streams_own_slices():
    """Each stream gets a slice of the library's array of its own: four streams are served (every call equal to the
    two-launch path), a fifth is refused without a launch, and after fck_fmha_fused_reset it is served."""
    lib = _lib.load()
    assert lib.fck_fmha_fused_reset(_stream()) == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(79)
    handles, keep = _other_streams(5)
    kv = gen.paged_kv([700, 31, 1500, 260], 4, 128, torch.bfloat16, g, 64)
    q = gen.randn((4, 1, 16, 128), torch.bfloat16, g)
    B, Hq, D, Hk, page, ns = 4, 16, 128, 4, 64, 3
    qd, kc, vc, sl, bt = dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"])
    _, o_ref = _run_both(lib, kv, q, ns)  # the current stream takes the first slice
    torch.cuda.synchronize()

    def fused_on(handle, out):
        return lib.fck_fmha_fwd_splitkv_fused(_vp(qd), _vp(kc), _vp(vc), None, _vp(out), None, None, _vp(sl), _vp(bt), None, B, 1, 0,
                                              Hq, Hk, D, D, 1, ns, bt.numel(), page, 1.0 / math.sqrt(D), -1, -1, 0, 4, handle)

    outs = [torch.full(q.shape, float("nan"), dtype=q.dtype, device=helpers.DEVICE) for _ in handles]
    torch.cuda.synchronize()  # the fills ran on the current stream; the calls below run on others
    # three more streams, launched back to back without a wait between them, twice each
    for _ in range(2):
        for h, o in zip(handles[:3], outs[:3]):
            assert fused_on(h, o) == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    for i in range(3):
        assert_bits_equal(outs[i], o_ref, f"stream {i + 1}")
    # all four slices are owned now
    assert fused_on(handles[3], outs[3]) == -2 and b"streams per GPU" in lib.fck_last_error()
    torch.cuda.synchronize()
    assert torch.isnan(outs[3].float()).all(), "a refused call must not launch"
    # the owners still work after the refusal
    assert fused_on(handles[0], outs[0]) == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    assert lib.fck_fmha_fused_reset(_stream()) == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    for h, o in zip(handles[3:], outs[3:]):
        assert fused_on(h, o) == 0, lib.fck_last_error().decode()
    torch.cuda.synchronize()
    for i in (3, 4):
        assert_bits_equal(outs[i], o_ref, f"stream {i + 1} after the reset")
    assert lib.fck_fmha_fused_reset(_stream()) == 0  # leave the table empty for whoever comes next
    torch.cuda.synchronize()
    del keep
