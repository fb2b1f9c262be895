"""GPU: one small problem for every kernel instantiation a call can reach.  The kernels are templates over the data type,
the head dim, the wave layout (packed query rows per workgroup, one or two KV heads) and a handful of flags (page
addressing, score modifiers, fp8 cache, padded head dims, equal-size splits); the other files reach most combinations in
passing, this one walks the grid on purpose, so that no instantiation first runs in a user's hands."""
import math

import pytest
import torch

from flashck_amd import _lib, generators as gen
from helpers import ATOL, assert_close, assert_fp8_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu

F8 = torch.float8_e4m3fn
DTYPES = [torch.bfloat16, torch.float16]


def _kernel():
    return _lib.load().fck_fmha_last_kernel().decode()


def _decode_cases():
    """(head dim, queries per sequence [x 4 heads per KV head = packed rows], KV heads per workgroup, page size, flags)"""
    out = []
    for d in (64, 128, 256):
        for sq in (1, 5, 12):                       # 4, 20, 48 packed rows: one 16-row block, two, four
            if d == 256 and sq == 12:
                continue                            # head dim 256 has one layout for everything above 16 rows
            for hg in (1, 2):
                if hg == 2 and (sq != 1 or d == 256):
                    continue                        # head pairs: at most 16 rows, head dim 64 / 128
                for page in (32, 16):               # tile-aligned pages / a lookup per cache row
                    for flags in ("plain", "mod", "kv8", "mod+kv8", "pad", "chunk"):
                        if flags == "pad" and hg == 2:
                            continue
                        if flags == "chunk" and (sq != 1 or d == 256 or page != 32):
                            continue
                        out.append((d, sq, hg, page, flags))
    return out


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("d,sq,hg,page,flags", _decode_cases())
def test_splitkv_instantiation(fmha, orc, dtype, d, sq, hg, page, flags):
    g = torch.Generator().manual_seed(d + sq + hg + page + len(flags))
    hk, hq, lens, ns = 2, 8, [70, 9, 33], 2
    dq, dv = (d - 8, d - 16) if flags == "pad" else (d, d)
    kv = gen.paged_kv(lens, hk, dq, dtype, g, page, dv=dv if dv != dq else None)
    q = gen.randn((len(lens), sq, hq, dq), dtype, g)
    kc, vc = kv["k_cache"], kv["v_cache"]
    kw = dict(scale=1.0 / math.sqrt(dq), mask_type=2, window=(-1, 0))
    okw = dict(kw)
    if "mod" in flags:
        kw["logits_soft_cap"] = okw["logits_soft_cap"] = 5.0
    if "kv8" in flags:
        kc, vc = (kc.float() / 0.03).clamp(-448, 448).to(F8), (vc.float() / 0.04).clamp(-448, 448).to(F8)
        kw.update(k_descale=0.03, v_descale=0.04)
        okw.update(k_descale=0.03, v_descale=0.04)
    variant = (3 if hg == 1 else 4) if flags == "chunk" else (hg if sq == 1 and d <= 128 and flags != "pad" else 0)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kc), dev(vc), ns, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                           decode_variant=variant, max_seqlen_k=max(lens) if flags == "chunk" else 0, **kw)
    name = _kernel()
    assert ("uniform_page" in name) == (page == 32) and ("head_pairs" in name) == (hg == 2), name
    assert ("kv_fp8" in name) == ("kv8" in flags) and ("score_mod" in name) == ("mod" in flags), name
    assert ("padded_head_dim" in name) == (flags == "pad") and ("equal_chunks" in name) == (flags == "chunk"), name
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    ro = orc.fmha_fwd(q, kc, vc, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **okw)
    assert_close(o, ro, ATOL[dtype], name)
    if flags != "chunk":
        ra, rl = orc.fmha_splitkv(q, kc, vc, ns, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **okw)
        assert_lse_close(lse_acc, rl, 2e-3, name + " lse_acc")
        assert_close(o_acc, ra, ATOL[dtype], name + " o_acc")


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("sq,hg", [(1, 1), (1, 2), (5, 1), (12, 1)])
@pytest.mark.parametrize("page", [32, 16])
def test_splitkv_instantiation_fp8_roles(fmha, orc, d, sq, hg, page):
    """e4m3 queries take the fp8-cache instantiations with modifiers (the identity here): every layout of those."""
    if (hg == 2 or sq == 12) and d == 256:
        pytest.skip("no such layout at head dim 256")
    g = torch.Generator().manual_seed(d + sq + hg + page)
    hk, hq, lens, ns = 2, 8, [70, 9, 33], 2
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page)
    q8 = lambda x, s: (x.float() / s).clamp(-448, 448).to(F8)
    Q, K, V = q8(torch.randn(len(lens), sq, hq, d, generator=g), 0.02), q8(kv["k_cache"], 0.03), q8(kv["v_cache"], 0.04)
    kw = dict(scale=0.02 / math.sqrt(d), k_descale=0.03, v_descale=0.04, mask_type=2, window=(-1, 0))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(Q), dev(K), dev(V), ns, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                           decode_variant=hg if sq == 1 and d <= 128 else 0, **kw)
    name = _kernel()
    assert "all_fp8" in name and ("head_pairs" in name) == (hg == 2) and ("uniform_page" in name) == (page == 32), name
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8)
    fine = orc.fmha_fwd(Q.float().to(torch.bfloat16), K, V, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw)
    assert_fp8_close(o, fine, name, outliers=1e-3)


def _prefill_cases():
    """(head dim, longest query run, page size, flags): the register-staged kernel takes short runs, pages that are not a
    multiple of 64, an elementwise bias, fp8 caches; the direct-to-LDS kernels everything else"""
    out = []
    for d in (64, 128, 256):
        for run in (40, 150):
            for page in (64, 16):
                for flags in ("plain", "alibi", "bias", "pad", "pad+alibi", "pad+bias", "kv8", "kv8+alibi"):
                    out.append((d, run, page, flags))
    return out


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("d,run,page,flags", _prefill_cases())
def test_prefill_instantiation(fmha, orc, dtype, d, run, page, flags):
    g = torch.Generator().manual_seed(d + run + page + len(flags))
    hk, hq = 2, 4
    lens_q = [run, 7]
    lens_k = [run + 30, 7]
    dq, dv = (d - 8, d - 16) if "pad" in flags else (d, d)
    kv = gen.paged_kv(lens_k, hk, dq, dtype, g, page, dv=dv if dv != dq else None)
    cq = torch.tensor([0, lens_q[0], sum(lens_q)], dtype=torch.int32)
    q = gen.randn((sum(lens_q), hq, dq), dtype, g)
    kc, vc = kv["k_cache"], kv["v_cache"]
    kw = dict(scale=1.0 / math.sqrt(dq), mask_type=2, window=(-1, 0))
    okw = dict(kw)
    if "alibi" in flags:
        s = torch.tensor([0.01, 0.02, 0.04, 0.08], dtype=torch.float32)
        kw["alibi_slopes"], okw["alibi_slopes"] = dev(s), s
    if "bias" in flags:
        b = (gen.randn((hq, sum(lens_q), max(lens_k)), dtype, g) * 1.5).contiguous()
        kw["bias"], okw["bias"] = dev(b), b
    if "kv8" in flags:
        kc, vc = (kc.float() / 0.03).clamp(-448, 448).to(F8), (vc.float() / 0.04).clamp(-448, 448).to(F8)
        kw.update(k_descale=0.03, v_descale=0.04)
        okw.update(k_descale=0.03, v_descale=0.04)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kc), dev(vc), dev(kv["seqlen_k"]), dev(kv["block_table"]), cu_seqlens_q=dev(cq), max_seqlen_q=max(lens_q), **kw)
    name = _kernel()
    fast = flags in ("plain", "alibi", "pad", "pad+alibi") and ((d <= 128 and run > 128) or (d == 256 and page == 64))
    assert name.startswith("prefill_kernel") != fast, name
    assert ("uniform_page" in name) == (page == 64) and ("padded_head_dim" in name) == ("pad" in flags) and ("kv_fp8" in name) == ("kv8" in flags), name
    ro = orc.fmha_fwd(q, kc, vc, seqstart_q=cq, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **okw)
    assert_close(o, ro, ATOL[dtype], name)


@pytest.mark.parametrize("out_dtype", [torch.float16, F8], ids=["fp16", "e4m3"])
@pytest.mark.parametrize("dv,rows", [(64, 170), (128, 90), (256, 45)])
def test_combine_many_rows_other_output_types(fmha, orc, out_dtype, dv, rows):
    """The 256-thread workgroups of the combine (taken when there are enough output rows) for fp16 and e4m3 outputs."""
    g = torch.Generator().manual_seed(dv + rows)
    B, H, ns = 3, 33, 3
    o_acc = torch.randn(B, H, ns, rows, dv, generator=g)
    lse = torch.randn(B, H, ns, rows, generator=g) * 2
    lse[2, 5, 1, :] = float("-inf")
    o = fmha.fmha_fwd_splitkv_combine(dev(lse), dev(o_acc), out_dtype)
    ref = orc.splitkv_combine(lse, o_acc, out_dtype)
    if out_dtype == F8:
        # same fp32 arithmetic up to the order of additions: a value may land on the other side of a rounding point
        assert_fp8_close(o, ref, "combine, many rows, e4m3", atol=0.0, outliers=0.0)
    else:
        assert_close(o, ref, 1e-2, "combine, many rows, fp16")
