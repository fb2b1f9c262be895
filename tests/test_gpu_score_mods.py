"""GPU parity of the score modifiers (elementwise bias, ALiBi, logits soft cap) against the CPU oracle, through the
*_attrs entry points of the C ABI: split-KV decode (paged, batch cache, group mode) and the prefill family (dense,
varlen, page list, block table)."""
import math

import pytest
import torch

from flashck_amd import _lib, generators as gen
import helpers
from helpers import ATOL, assert_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu

SLOPES8 = [2.0 ** (-(i + 1)) for i in range(8)]


def mods(kind, dtype, g, B, Hq, rows, cols, group=False):
    """(oracle kwargs, device kwargs) for one modifier kind; bias shapes cover the reference's ranks 0, 1, 2"""
    if kind == "cap":
        return dict(logits_soft_cap=1.7), dict(logits_soft_cap=1.7)
    if kind.startswith("alibi"):
        sl = torch.tensor([SLOPES8[h % 8] for h in range(Hq)], dtype=torch.float32)
        if kind == "alibi_b":
            sl = torch.stack([sl * (1 + 0.5 * b) for b in range(B)]).contiguous()
        return dict(alibi_slopes=sl), dict(alibi_slopes=dev(sl))
    rank = int(kind[-1])
    if group:
        shape = (1 if rank == 0 else Hq, rows, cols)
    else:
        shape = (B if rank == 2 else 1, 1 if rank == 0 else Hq, rows, cols)
    bias = (gen.randn(shape, dtype, g) * 1.5).contiguous()
    extra = {}
    if kind.startswith("biascap"):
        extra = dict(logits_soft_cap=3.0)
    return dict(bias=bias, **extra), dict(bias=dev(bias), **extra)


KINDS = ["cap", "alibi_h", "alibi_b", "bias0", "bias1", "bias2", "biascap1"]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hk,d,page,ns", [(8, 2, 128, 128, 3), (16, 8, 64, 16, 2), (4, 4, 256, 64, 1)])
def test_paged_decode_with_modifiers(fmha, orc, dtype, kind, hq, hk, d, page, ns):
    w = gen.workload_paged_decode(seed=21 + hq + d, batch=3, hq=hq, hk=hk, head_dim=d, min_len=1, max_len=500, page_size=page,
                                  dtype=dtype)
    g = torch.Generator().manual_seed(5)
    okw, dkw = mods(kind, dtype, g, 3, hq, 1, max(w["lens"]))
    q, kc, vc, bt, sl = (dev(w[k]) for k in ("q", "k_cache", "v_cache", "block_table", "seqlen_k"))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=sl, block_table=bt, scale=w["scale"], **dkw)
    assert _lib.load().fck_fmha_last_kernel().endswith(b"score_mod>")
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    torch.cuda.synchronize()
    kw = dict(seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"], **okw)
    ro_acc, rlse_acc = orc.fmha_splitkv(w["q"], w["k_cache"], w["v_cache"], ns, **kw)
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], **kw)
    assert_lse_close(lse_acc, rlse_acc, what="lse_acc")
    assert_close(o_acc, ro_acc, ATOL[dtype], "o_acc")
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("mask_type,window", [(2, (-1, 0)), (1, (-1, 0)), (2, (9, 2)), (1, (4, 4)), (0, (-1, -1))])
def test_multi_query_decode_masks_with_modifiers(fmha, orc, kind, mask_type, window):
    """Several query rows per sequence (GQA rows packed into one tile) under every mask family: the ALiBi mode follows
    the mask (vertical for causal windows, else the mask's diagonal), bias rows follow the query row."""
    g = torch.Generator().manual_seed(31)
    dtype, sq, hq, hk, d = torch.bfloat16, 5, 8, 2, 128
    lens = [5, 40, 133]
    kv = gen.paged_kv(lens, hk, d, dtype, g, 64)
    qh = gen.randn((len(lens), sq, hq, d), dtype, g)
    okw, dkw = mods(kind, dtype, g, len(lens), hq, sq, max(lens))
    q, kc, vc, bt, sl = dev(qh), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["block_table"]), dev(kv["seqlen_k"])
    scale = 1 / math.sqrt(d)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, kc, vc, 2, seqlen_k=sl, block_table=bt, scale=scale, mask_type=mask_type,
                                           window=window, **dkw)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale,
                      mask_type=mask_type, window=window, **okw)
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("kind", ["cap", "alibi_b", "bias1"])
def test_group_mode_decode_with_modifiers(fmha, orc, kind):
    g = torch.Generator().manual_seed(41)
    dtype, hq, hk, d = torch.float16, 4, 2, 64
    lens_q, lens_k = [2, 1, 4], [50, 17, 90]
    cuq = torch.tensor([0, 2, 3, 7], dtype=torch.int32)
    cuk = torch.tensor([0, 50, 67, 157], dtype=torch.int32)
    qh, kh, vh = gen.randn((7, hq, d), dtype, g), gen.randn((157, hk, d), dtype, g), gen.randn((157, hk, d), dtype, g)
    okw, dkw = mods(kind, dtype, g, 3, hq, 7, max(lens_k), group=True)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(qh), dev(kh), dev(vh), 3, cu_seqlens_q=dev(cuq), cu_seqlens_k=dev(cuk), max_seqlen_q=4,
                                           mask_type=2, window=(-1, 0), **dkw)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype, cu_seqlens_q=dev(cuq))
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, kh, vh, seqstart_q=cuq, seqstart_k=cuk, mask_type=2, window=(-1, 0), **okw)
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("d,mask_type,window", [(64, 0, (-1, -1)), (128, 2, (-1, 0)), (256, 1, (20, 3))])
def test_dense_forward_with_modifiers(fmha, orc, dtype, kind, d, mask_type, window):
    g = torch.Generator().manual_seed(51 + d)
    B, sq, sk, hq, hk = 2, 150, 210, 4, 2
    qh, kh, vh = gen.randn((B, sq, hq, d), dtype, g), gen.randn((B, sk, hk, d), dtype, g), gen.randn((B, sk, hk, d), dtype, g)
    okw, dkw = mods(kind, dtype, g, B, hq, sq, sk)
    o = fmha.fmha_fwd(dev(qh), dev(kh), dev(vh), mask_type=mask_type, window=window, **dkw)
    # an elementwise bias is read by the register-staged kernel only; ALiBi and the soft cap run on the kernel the plain
    # call would take (150 query rows: ping-pong at head dim <= 128, direct-to-LDS at 256)
    fast = b"prefill_dma_kernel" if d == 256 else b"prefill_pp_kernel"
    want = (b"prefill_kernel" if kind.startswith("bias") else fast) + b"<uniform_page,score_mod>"
    assert _lib.load().fck_fmha_last_kernel() == want
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, kh, vh, mask_type=mask_type, window=window, **okw)
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("kind", ["cap", "alibi_h", "bias1", "bias0"])
def test_varlen_forward_with_modifiers(fmha, orc, kind):
    g = torch.Generator().manual_seed(61)
    dtype, hq, hk, d = torch.bfloat16, 4, 4, 128
    lens = [1, 130, 77]
    cu = torch.tensor([0, 1, 131, 208], dtype=torch.int32)
    qh, kh, vh = gen.randn((208, hq, d), dtype, g), gen.randn((208, hk, d), dtype, g), gen.randn((208, hk, d), dtype, g)
    okw, dkw = mods(kind, dtype, g, 3, hq, 208, max(lens), group=True)
    o = fmha.fmha_fwd_varlen(dev(qh), dev(kh), dev(vh), dev(cu), dev(cu), 130, mask_type=2, window=(-1, 0), **dkw)
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, kh, vh, seqstart_q=cu, seqstart_k=cu, mask_type=2, window=(-1, 0), **okw)
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("kind", ["cap", "alibi_b", "bias1"])
@pytest.mark.parametrize("page", [128, 48])
def test_batch_prefill_with_modifiers(fmha, orc, kind, page):
    """Page-list prefill: long enough (> 128 rows) that the plain call would take the ping-pong kernel, so this also
    checks that a call with modifiers is routed to the kernel that applies them."""
    dtype = torch.bfloat16
    w = gen.workload_varlen_prefill(seed=71, batch=3, hq=4, hk=2, head_dim=128, min_len=20, max_len=300, page_size=page, dtype=dtype)
    g = torch.Generator().manual_seed(6)
    tq = sum(w["lens"])
    okw, dkw = mods(kind, dtype, g, 3, 4, tq, max(w["lens"]), group=True)
    a = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], **dkw)
    assert _lib.load().fck_fmha_last_kernel().endswith(b"score_mod>")
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"],
                      mask_type=2, window=(-1, 0), **okw)
    assert_close(o, ro, ATOL[dtype], "o")


@pytest.mark.parametrize("kind", ["cap", "alibi_h", "bias2"])
def test_pagedkv_prefill_with_modifiers(fmha, orc, kind):
    g = torch.Generator().manual_seed(81)
    dtype, sq, hq, hk, d = torch.float16, 33, 4, 2, 128
    lens = [33, 100, 64]
    kv = gen.paged_kv(lens, hk, d, dtype, g, 64)
    qh = gen.randn((3, sq, hq, d), dtype, g)
    okw, dkw = mods(kind, dtype, g, 3, hq, sq, max(lens))
    o = fmha.fmha_fwd_pagedkv(dev(qh), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), **dkw)
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=2,
                      window=(-1, 0), **okw)
    assert_close(o, ro, ATOL[dtype], "o")


def test_modifier_arguments_are_validated(fmha):
    g = torch.Generator().manual_seed(1)
    q, k, v = (dev(gen.randn((1, 4, 4, 64), torch.float16, g)) for _ in range(3))
    with pytest.raises(ValueError):
        fmha.fmha_fwd(q, k, v, bias=dev(gen.randn((1, 4, 3, 4), torch.float16, g)))          # wrong row count
    with pytest.raises(TypeError):
        fmha.fmha_fwd(q, k, v, bias=dev(gen.randn((1, 4, 4, 4), torch.bfloat16, g)))         # wrong dtype
    with pytest.raises(ValueError):
        fmha.fmha_fwd(q, k, v, alibi_slopes=torch.ones(3, dtype=torch.float32, device=helpers.DEVICE))  # wrong head count
    with pytest.raises(ValueError):
        fmha.fmha_fwd(q, k, v, logits_soft_cap=-1.0)
    with pytest.raises(NotImplementedError):                                                 # ALiBi has no diagonal for GENERIC
        fmha.fmha_fwd(q, k, v, mask_type=3, window=(1, 1), alibi_slopes=torch.ones(4, dtype=torch.float32, device=helpers.DEVICE))
    # a raw bias pointer without attributes is refused by the C ABI (nothing says what it holds)
    import ctypes
    lib = _lib.load()
    o = torch.empty_like(q)
    rc = lib.fck_fmha_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), q.data_ptr(), o.data_ptr(), None, None, None, 1, 4, 4, 4, 4, 64, 64,
                          4, 0.125, -1, -1, 0, 3, None)
    assert rc == -2 and b"fck_fmha_attrs" in lib.fck_last_error()
    del ctypes


def quantise_cache(kv, k_descale, v_descale):
    """fp8 (e4m3) copies of a paged cache with static per-tensor scales; unused slots stay NaN"""
    k8 = (kv["k_cache"].float() / k_descale).to(torch.float8_e4m3fn)
    v8 = (kv["v_cache"].float() / v_descale).to(torch.float8_e4m3fn)
    return k8, v8


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hk,d,page,ns,batch", [(8, 2, 128, 128, 3, 3), (32, 8, 128, 128, 4, 20), (16, 8, 64, 64, 2, 3),
                                                   (4, 4, 256, 64, 2, 2), (8, 2, 128, 48, 2, 3)])
def test_paged_decode_fp8_cache(fmha, orc, dtype, hq, hk, d, page, ns, batch):
    """K/V stored as e4m3 bytes with static scales; q, the probabilities and the output keep the 16-bit type.  The
    20-sequence case fills the grid, so it takes the two-heads-per-workgroup variant; page 48 the per-row lookup."""
    w = gen.workload_paged_decode(seed=91 + hq + d, batch=batch, hq=hq, hk=hk, head_dim=d, min_len=1, max_len=600, page_size=page,
                                  dtype=dtype)
    kd, vd = 0.03, 0.025
    k8, v8 = quantise_cache(w, kd, vd)
    q, bt, sl = dev(w["q"]), dev(w["block_table"]), dev(w["seqlen_k"])
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, dev(k8), dev(v8), ns, seqlen_k=sl, block_table=bt, scale=w["scale"], k_descale=kd,
                                           v_descale=vd)
    assert b"kv_fp8" in _lib.load().fck_fmha_last_kernel()
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    torch.cuda.synchronize()
    kw = dict(seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"], k_descale=kd, v_descale=vd)
    ro_acc, rlse_acc = orc.fmha_splitkv(w["q"], k8, v8, ns, **kw)
    ro = orc.fmha_fwd(w["q"], k8, v8, **kw)
    assert_lse_close(lse_acc, rlse_acc, what="lse_acc")
    assert_close(o_acc, ro_acc, ATOL[dtype], "o_acc")
    assert_close(o, ro, ATOL[dtype], "o")


def test_multi_query_decode_fp8_cache_with_alibi(fmha, orc):
    g = torch.Generator().manual_seed(95)
    dtype, sq, hq, hk, d = torch.bfloat16, 6, 8, 2, 128
    lens = [6, 70, 200]
    kv = gen.paged_kv(lens, hk, d, dtype, g, 64)
    k8, v8 = quantise_cache(kv, 0.04, 0.04)
    qh = gen.randn((3, sq, hq, d), dtype, g)
    okw, dkw = mods("alibi_h", dtype, g, 3, hq, sq, max(lens))
    scale = 1 / math.sqrt(d)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(qh), dev(k8), dev(v8), 2, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                           scale=scale, mask_type=2, window=(-1, 0), k_descale=0.04, v_descale=0.04, **dkw)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    torch.cuda.synchronize()
    ro = orc.fmha_fwd(qh, k8, v8, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale, mask_type=2, window=(-1, 0),
                      k_descale=0.04, v_descale=0.04, **okw)
    assert_close(o, ro, ATOL[dtype], "o")


def test_fp8_cache_is_refused_where_no_kernel_reads_it(fmha):
    import ctypes
    lib = _lib.load()
    at = _lib.Attrs()
    at.size, at.kv_dtype = ctypes.sizeof(_lib.Attrs), 1
    x = torch.zeros(1, 4, 4, 128, dtype=torch.float16, device=helpers.DEVICE)
    # head dims the kernels pad (qk 64, v 128) do not combine with an fp8 cache
    rc = lib.fck_fmha_fwd_attrs(x.data_ptr(), x.data_ptr(), x.data_ptr(), None, x.data_ptr(), None, None, None, 1, 4, 4, 4, 4, 64, 128,
                                4, 0.125, -1, -1, 0, 3, ctypes.byref(at), None)
    assert rc == -2 and b"fp8 K/V cache needs" in lib.fck_last_error()
    at.kv_dtype = 2   # only e4m3 (FLOAT8 = 1) is a cache type
    rc = lib.fck_fmha_fwd_attrs(x.data_ptr(), x.data_ptr(), x.data_ptr(), None, x.data_ptr(), None, None, None, 1, 4, 4, 4, 4, 128, 128,
                                4, 0.125, -1, -1, 0, 3, ctypes.byref(at), None)
    assert rc == -2 and b"kv_dtype 2" in lib.fck_last_error()
