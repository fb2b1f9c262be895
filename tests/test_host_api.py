"""CPU-only checks of the boundary: the built library exports every symbol the header declares, argument validation
answers with error codes and messages before any launch, and the Python operators validate like the reference's."""
import ctypes
import os
import re

import pytest
import torch

from flashck_amd import _lib
from flashck_amd.ops import fmha
from flashck_amd.utils import FlashCKOperationType, get_flashck_functions, is_available

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flashck", "fmha", "fmha_c_api.h")


def declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"FCK_EXPORT\s+[\w\s\*]+?\b(fck_\w+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 10
    assert set(names) == set(_lib.SIGNATURES), "ctypes signature table and header disagree"
    for n in names:
        assert getattr(lib, n) is not None


def test_registry_has_fmha():
    assert is_available(FlashCKOperationType.FMHA.value)
    fns = get_flashck_functions("fmha")
    for k in ("forward", "forward_splitkv", "forward_splitkv_combine", "forward_appendkv", "batch_prefill", "forward_pagedkv"):
        assert callable(fns[k])
    assert not is_available(FlashCKOperationType.LAYER_NORM.value)


def test_error_codes_without_a_gpu():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    # unsupported dtype
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 7, None)
    assert rc == -2 and b"dtype" in lib.fck_last_error()
    # Hq not a multiple of Hk
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 3, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -1 and b"multiple" in lib.fck_last_error()
    # unsupported head dims: not a multiple of 8, beyond 256
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 84, 84, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -2 and b"head_dim" in lib.fck_last_error()
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 264, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -2 and b"head_dim" in lib.fck_last_error()
    # null pointer
    rc = lib.fck_fmha_fwd(None, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -1 and b"null" in lib.fck_last_error()
    # bias is declared by the signature but has no kernel
    rc = lib.fck_fmha_fwd(p, p, p, p, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -2 and b"bias" in lib.fck_last_error()
    # misaligned pointer
    q = ctypes.c_void_p(p.value + 2)
    rc = lib.fck_fmha_fwd(q, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None)
    assert rc == -1 and b"aligned" in lib.fck_last_error()
    # split-KV: bad split count, paged cache without key counts
    rc = lib.fck_fmha_fwd_splitkv(p, p, p, None, p, p, None, None, None, None, None, 1, 1, 8, 2, 2, 64, 64, 1, 0, 0, 0,
                                  0.125, -1, -1, 0, 4, None)
    assert rc == -1 and b"num_splits" in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_splitkv(p, p, p, None, p, p, None, None, None, p, None, 1, 1, 8, 2, 2, 64, 64, 1, 2, 4, 16,
                                  0.125, -1, -1, 0, 4, None)
    assert rc == -1 and b"key counts" in lib.fck_last_error()
    # combine: bad head dim; appendkv: odd rotary_dim
    rc = lib.fck_fmha_fwd_splitkv_combine(p, p, p, None, 1, 1, 2, 100, 1, 2, 4, None)
    assert rc == -2
    rc = lib.fck_fmha_fwd_appendkv(None, p, p, p, p, p, None, 1, p, p, 31, 2, 1, p, 4, 16, None, 0, 1, 2, 2, 64, 64, 4, None)
    assert rc == -1 and b"rotary_dim" in lib.fck_last_error()
    # mask type out of range
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 9, 4, None)
    assert rc == -1 and b"mask_type" in lib.fck_last_error()


def test_workspace_bytes_and_heuristic():
    lib = _lib.load()
    # o_acc [B,Hq,ns,sq,Dv] fp32 + lse_acc [B,Hq,ns,sq] fp32
    assert lib.fck_fmha_splitkv_workspace_bytes(4, 64, 1, 128, 8) == 4 * 64 * 8 * 1 * 128 * 4 + 4 * 64 * 8 * 4
    assert lib.fck_fmha_splitkv_workspace_bytes(0, 64, 1, 128, 8) == 0
    # long context, few sequences: split; many workgroups already or short context: do not
    assert fmha.num_splits_heuristic(4, 64, 8, 1, 32768, 128, 256) >= 8
    assert fmha.num_splits_heuristic(256, 32, 8, 1, 4096, 128, 256) == 1
    assert fmha.num_splits_heuristic(1, 8, 8, 1, 200, 128, 256) == 1
    for args in [(1, 8, 1, 1, 10 ** 6, 128, 256), (32, 32, 8, 1, 4096, 128, 256)]:
        assert 1 <= fmha.num_splits_heuristic(*args) <= 128
    # sizes no launch could have answer 1 (batch * kv heads used to wrap to zero here, and the next line divided by it)
    assert lib.fck_fmha_num_splits_heuristic(1 << 31, 2, 1 << 62, 96, (1 << 31) - 1, 1, 1 << 31) == 1
    assert lib.fck_fmha_num_splits_heuristic(4, 2, 8, 1, 4096, 128, 256) == 1      # more KV heads than query heads
    assert lib.fck_fmha_num_splits_heuristic(1 << 40, 8, 8, 1, 4096, 128, 256) == 1


def test_python_validation_mirrors_reference_errors():
    q = torch.zeros(1, 4, 2, 64, dtype=torch.float16)
    with pytest.raises(TypeError):
        fmha.fmha_fwd("q", q, q)
    with pytest.raises(ValueError):   # CPU tensors never reach the GPU path and there is no fallback
        fmha.fmha_fwd(q, q, q)
    with pytest.raises(TypeError):
        fmha.fmha_fwd_splitkv_combine(torch.zeros(1, 2, 1, 4), torch.zeros(1, 2, 1, 4, 64), torch.float32)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libflashck_fmha.so"))
    with pytest.raises(_lib.FlashCKLibraryError):
        _lib.load()


@pytest.fixture()
def host_ops(monkeypatch):
    """The Python operators with the GPU-residency check off and the C call recorded instead of made, so that the
    shape / dtype validation in front of the C ABI can be exercised with CPU tensors."""
    calls = []
    monkeypatch.setattr(fmha.fmha, "_REQUIRE_GPU_TENSORS", False)
    monkeypatch.setattr(fmha.fmha, "_call", lambda name, *a: calls.append(name))
    monkeypatch.setattr(fmha.fmha, "_stream", lambda: None)
    return calls


def test_caller_supplied_buffers_are_validated(host_ops):
    T = torch.bfloat16
    B, Hq, Hk, D, P, ns = 2, 4, 2, 64, 16, 3
    q = torch.zeros(B, 1, Hq, D, dtype=T)
    kc, vc = torch.zeros(8, P, Hk, D, dtype=T), torch.zeros(8, P, Hk, D, dtype=T)
    sl = torch.full((B,), 20, dtype=torch.int32)
    bt = torch.zeros(B, 4, dtype=torch.int32)
    o_acc, lse_acc = torch.zeros(B, Hq, ns, 1, D), torch.zeros(B, Hq, ns, 1)
    fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, o_acc=o_acc, lse_acc=lse_acc)
    assert host_ops == ["fck_fmha_fwd_splitkv"]
    # a workspace laid out for another split count would be written out of bounds
    with pytest.raises(ValueError, match="o_acc must have shape"):
        fmha.fmha_fwd_splitkv(q, kc, vc, ns + 1, seqlen_k=sl, block_table=bt, o_acc=o_acc, lse_acc=lse_acc)
    with pytest.raises(ValueError, match="lse_acc must have shape"):
        fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, o_acc=o_acc, lse_acc=lse_acc[:, :, :2].contiguous())
    with pytest.raises(TypeError, match="o_acc"):
        fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, o_acc=o_acc.half(), lse_acc=lse_acc)
    with pytest.raises(ValueError, match="together"):
        fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, o_acc=o_acc)
    # k with another head dim, v that disagrees with k, wrong rank
    with pytest.raises(ValueError, match="head dim"):
        fmha.fmha_fwd_splitkv(q, torch.zeros(8, P, Hk, 128, dtype=T), vc, ns, seqlen_k=sl, block_table=bt)
    with pytest.raises(ValueError, match="does not match k"):
        fmha.fmha_fwd_splitkv(q, kc, torch.zeros(8, P, 1, D, dtype=T), ns, seqlen_k=sl, block_table=bt)
    with pytest.raises(ValueError, match="dimensions"):
        fmha.fmha_fwd_splitkv(q, kc[0], vc[0], ns, seqlen_k=sl, block_table=bt)
    # decode with a caller-owned workspace and num_splits = 0: the workspace's split count is the one used
    del host_ops[:]
    fmha.fmha_decode_paged(q, kc, vc, sl, bt, num_splits=0, workspace=(o_acc, lse_acc))
    assert host_ops == ["fck_fmha_fwd_splitkv", "fck_fmha_fwd_splitkv_combine"]
    with pytest.raises(ValueError, match="o_acc must have shape"):
        fmha.fmha_decode_paged(q, kc, vc, sl, bt, num_splits=5, workspace=(o_acc, lse_acc))
    # out= of every operator
    with pytest.raises(ValueError, match="out must have shape"):
        fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, T, out=torch.zeros(B, 1, Hq, D - 8, dtype=T))
    with pytest.raises(TypeError, match="out"):
        fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, T, out=torch.zeros(B, 1, Hq, D, dtype=torch.float16))
    qd = torch.zeros(B, 5, Hq, D, dtype=T)
    kd = torch.zeros(B, 7, Hk, D, dtype=T)
    with pytest.raises(ValueError, match="out must have shape"):
        fmha.fmha_fwd(qd, kd, kd, out=torch.zeros(B, 4, Hq, D, dtype=T))
    with pytest.raises(ValueError, match="out must have shape"):
        fmha.fmha_fwd_pagedkv(qd, kc, vc, sl, bt, out=torch.zeros(B, 5, Hq, 2 * D, dtype=T))
    cu = torch.tensor([0, 3, 5], dtype=torch.int32)
    qp = torch.zeros(5, Hq, D, dtype=T)
    with pytest.raises(ValueError, match="out must have shape"):
        fmha.fmha_batch_prefill(qp, kc, vc, cu, torch.tensor([0, 1, 2], dtype=torch.int32),
                                torch.tensor([0, 1], dtype=torch.int32), max_seqlen_q=3, out=torch.zeros(4, Hq, D, dtype=T))
    with pytest.raises(ValueError, match="out must have shape"):
        fmha.fmha_fwd_varlen(qp, torch.zeros(9, Hk, D, dtype=T), torch.zeros(9, Hk, D, dtype=T), cu, cu, 3,
                             out=torch.zeros(5, Hq, D + 8, dtype=T))
    # appendkv: caches that do not match the new tokens
    kn = torch.zeros(B, 1, Hk, D, dtype=T)
    with pytest.raises(ValueError, match="do not match knew"):
        fmha.fmha_fwd_appendkv(None, kc, torch.zeros(8, P, Hk, 32, dtype=T), kn, kn, sl, block_table=bt)


def test_validate_paged_arguments_are_checked_before_any_launch():
    """fck_fmha_validate_paged: argument errors come back as a status, without a GPU."""
    import ctypes
    lib = _lib.load()
    buf = (ctypes.c_int32 * 8)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = lib.fck_fmha_validate_paged(p, p, 2, None, None, None, 0, 4, 16, p, None)          # batch 0
    assert rc == -1 and b"positive" in lib.fck_last_error()
    rc = lib.fck_fmha_validate_paged(p, p, 2, p, p, None, 1, 4, 16, p, None)                # table and list
    assert rc == -1 and b"either" in lib.fck_last_error()
    rc = lib.fck_fmha_validate_paged(None, None, 0, None, None, None, 1, 4, 16, p, None)    # neither
    assert rc == -1 and b"either" in lib.fck_last_error()
    rc = lib.fck_fmha_validate_paged(None, p, 2, None, None, None, 1, 4, 16, p, None)       # table without lengths
    assert rc == -1 and b"seqlen_k" in lib.fck_last_error()
    rc = lib.fck_fmha_validate_paged(p, p, 2, None, None, None, 1, 4, 16, None, None)       # no counters
    assert rc == -1 and b"error_counts" in lib.fck_last_error()


def test_fp8_roles_are_validated_before_any_launch():
    """dtype FLOAT8 (1): what the all-fp8 roles do not cover is refused with FCK_ERR_UNSUPPORTED, bad scales with
    FCK_ERR_INVALID_ARGUMENT; no GPU is needed to get that far."""
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    FP8 = 1
    # stored head dims other than 64 / 128 / 256, or unequal
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 96, 96, 8, 0.125, -1, -1, 0, FP8, None)
    assert rc == -2 and b"e4m3" in lib.fck_last_error()
    rc = lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 128, 64, 8, 0.125, -1, -1, 0, FP8, None)
    assert rc == -2 and b"e4m3" in lib.fck_last_error()
    # scales
    at = _lib.Attrs()
    at.size = ctypes.sizeof(_lib.Attrs)
    at.o_scale = -1.0
    rc = lib.fck_fmha_fwd_attrs(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, FP8, ctypes.byref(at), None)
    assert rc == -1 and b"o_scale" in lib.fck_last_error()
    at.o_scale, at.kv_dtype = 0.0, 4
    rc = lib.fck_fmha_fwd_attrs(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, FP8, ctypes.byref(at), None)
    assert rc == -2 and b"kv_dtype" in lib.fck_last_error()
    # the split-KV partial results are fp32: an output scale has nowhere to go
    at = _lib.Attrs()
    at.size = ctypes.sizeof(_lib.Attrs)
    at.o_scale = 2.0
    rc = lib.fck_fmha_fwd_splitkv_attrs(p, p, p, None, p, p, None, None, None, None, None, 1, 1, 8, 2, 2, 64, 64, 1, 2, 0, 0, 0.125, -1, -1,
                                        0, FP8, ctypes.byref(at), None)
    assert rc == -2 and b"o_scale" in lib.fck_last_error()
    # the one-launch entry point and appendKV have no e4m3 kernels
    rc = lib.fck_fmha_fwd_splitkv_fused(p, p, p, None, p, None, None, None, None, None, 1, 1, 8, 2, 2, 64, 64, 1, 2, 0, 0, 0.125, -1, -1, 0,
                                        FP8, None)
    assert rc == -2 and b"e4m3" in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_appendkv(None, p, p, p, p, p, None, 1, None, None, 0, 0, 0, None, 0, 0, None, 0, 1, 2, 2, 64, 64, FP8, None)
    assert rc == -2
    # an unknown dtype still names the ones there are
    rc = lib.fck_fmha_fwd_splitkv_combine(p, p, p, None, 1, 1, 2, 64, 1, 2, 9, None)
    assert rc == -2 and b"FLOAT8" in lib.fck_last_error()


def test_sizes_beyond_32_bits_are_refused_not_truncated():
    """2^32 + 1 sequences must not run as 1 sequence: counts, lengths and strides the kernels keep in 32 bits are range-checked."""
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    big = (1 << 32) + 1
    msg = b"beyond 32 bits"
    assert lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, big, 8, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None) == -1 and msg in lib.fck_last_error()
    assert lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, big, 8, 2, 2, 64, 64, 8, 0.125, -1, -1, 0, 4, None) == -1 and msg in lib.fck_last_error()
    assert lib.fck_fmha_fwd(p, p, p, None, p, None, None, None, 1, 8, 8, 2, 2, 64, 64, big, 0.125, -1, -1, 0, 4, None) == -1 and msg in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_splitkv(p, p, p, None, p, p, None, None, None, None, None, 1, 1, big, 2, 2, 64, 64, 1, 2, 0, 0, 0.125, -1, -1, 0, 4, None)
    assert rc == -1 and msg in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_splitkv(p, p, p, None, p, p, None, None, p, p, None, 1, 1, 0, 2, 2, 64, 64, 1, 2, 4, big, 0.125, -1, -1, 0, 4, None)
    assert rc == -1 and msg in lib.fck_last_error()
    assert lib.fck_fmha_fwd_splitkv_combine(p, p, p, None, 1, big, 2, 64, 1, 2, 4, None) == -1 and msg in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_appendkv(None, p, p, p, p, p, None, big, None, None, 0, 0, 0, p, 4, 16, None, 0, 1, 2, 2, 64, 64, 4, None)
    assert rc == -1 and msg in lib.fck_last_error()
    rc = lib.fck_fmha_batch_prefill(p, p, p, p, p, p, p, None, big, 16, 1, 2, 2, 64, 64, 8, 0.125, -1, 0, 2, 4, None)
    assert rc == -1 and msg in lib.fck_last_error()
    rc = lib.fck_fmha_fwd_pagedkv(p, p, p, p, None, p, p, big, 16, 1, 8, 2, 2, 64, 64, 8, 0.125, -1, 0, 2, 4, None)
    assert rc == -1 and msg in lib.fck_last_error()
