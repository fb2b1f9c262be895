"""Host logic of the decode step and of the nn modules, with the three kernels replaced by the CPU oracle.

What is checked here is the composition: which operator is called with which lengths, mask, window and workspace views.
The kernels themselves are checked against the oracle in the GPU tests.
"""
import math

import pytest
import torch

from flashck_amd import generators as gen
from flashck_amd.ops.fmha import fmha as F
from helpers import assert_bits_equal, assert_close


@pytest.fixture()
def cpu_ops(monkeypatch, orc):
    """Route the operators the decode step composes to the oracle; record the calls."""
    calls = []

    def appendkv(q, k_cache, v_cache, knew, vnew, seqlen_k, *, cu_seqlens_knew=None, max_seqlen_knew=0, rotary_cos=None,
                 rotary_sin=None, rope_mode=F.ROPE_NONE, has_mask=True, block_table=None, cache_batch_idx=None, k_descale=1.0,
                 v_descale=1.0):
        calls.append(("appendkv", dict(max_seqlen_knew=max_seqlen_knew, rope_mode=rope_mode, has_mask=has_mask)))
        cu = cu_seqlens_knew
        if cu is None:
            B, n = knew.shape[:2]
            cu = torch.arange(0, (B + 1) * n, n, dtype=torch.int32)
            q, knew, vnew = q.view(-1, *q.shape[2:]), knew.view(-1, *knew.shape[2:]), vnew.view(-1, *vnew.shape[2:])
        orc.appendkv(q, k_cache, v_cache, knew, vnew, seqlen_k, cu, cos=rotary_cos, sin=rotary_sin, rope_mode=rope_mode,
                     has_mask=has_mask, block_table=block_table)

    def splitkv(q, k, v, num_splits, *, seqlen_k=None, block_table=None, cache_batch_idx=None, cu_seqlens_q=None,
                cu_seqlens_k=None, max_seqlen_q=0, scale=0.0, mask_type=F.MASK_NONE, window=(-1, -1), o_acc=None,
                lse_acc=None, decode_variant=0, k_descale=1.0, v_descale=1.0, max_seqlen_k=0):
        assert decode_variant == 0   # nothing is cached in these tests: the library picks the kernel variant
        calls.append(("splitkv", dict(num_splits=num_splits, mask_type=mask_type, window=tuple(window),
                                      max_seqlen_q=max_seqlen_q, seqlen_k=seqlen_k.clone(), o_acc=o_acc, lse_acc=lse_acc)))
        ro, rl = orc.fmha_splitkv(q, k, v, num_splits, seqstart_q=cu_seqlens_q, seqlen_k=seqlen_k.contiguous(),
                                  block_table=block_table, scale=scale or 1.0 / math.sqrt(q.shape[-1]),
                                  mask_type=mask_type, window=window)
        assert o_acc.shape == ro.shape and lse_acc.shape == rl.shape
        o_acc.copy_(ro)
        lse_acc.copy_(rl)
        return o_acc, lse_acc

    def combine(lse_acc, o_acc, dtype, cu_seqlens_q=None, max_seqlen_q=0, out=None):
        calls.append(("combine", dict(max_seqlen_q=max_seqlen_q)))
        o = orc.splitkv_combine(lse_acc.contiguous(), o_acc.contiguous(), dtype, seqstart_q=cu_seqlens_q)
        if out is not None:
            out.copy_(o)
            return out
        return o

    def heuristic(batch, hq, hk, sq, max_sk, d, num_cu=0):
        calls.append(("heuristic", dict(batch=batch, hq=hq, hk=hk, sq=sq, max_sk=max_sk, d=d)))
        return 3

    monkeypatch.setattr(F, "fmha_fwd_appendkv", appendkv)
    monkeypatch.setattr(F, "fmha_fwd_splitkv", splitkv)
    monkeypatch.setattr(F, "fmha_fwd_splitkv_combine", combine)
    monkeypatch.setattr(F, "num_splits_heuristic", heuristic)
    return calls


def _expected(orc, w, rope_mode, window_left=-1):
    q, kc, vc = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    orc.appendkv(q, kc, vc, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos=w["rotary_cos"],
                 sin=w["rotary_sin"], rope_mode=rope_mode, has_mask=True, block_table=w["block_table"])
    sl = (w["seqlen_k"] + torch.tensor(w["new"], dtype=torch.int32)).contiguous()
    o = orc.fmha_fwd(q, kc, vc, seqstart_q=w["cu_seqlens_knew"], seqlen_k=sl, block_table=w["block_table"],
                     scale=w["scale"], mask_type=2, window=(window_left, 0))
    return o, q, kc, vc, sl


def _workload(seed=7, **kw):
    args = dict(seed=seed, batch=5, hq=8, hk=2, head_dim=64, min_len=0, max_len=200, max_new=6, page_size=16)
    args.update(kw)
    return gen.workload_appendkv_decode(**args)


@pytest.mark.parametrize("window_left", [-1, 37])
def test_packed_step_equals_append_then_causal_attention(cpu_ops, orc, window_left):
    w = _workload()
    q, kc, vc = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    ws = F.DecodeWorkspace()
    o, sl_new = F.fmha_decode_step(q, w["knew"], w["vnew"], kc, vc, w["seqlen_k"], w["block_table"],
                                   cu_seqlens_knew=w["cu_seqlens_knew"], max_seqlen_knew=w["max_new"],
                                   rotary_cos=w["rotary_cos"], rotary_sin=w["rotary_sin"], rope_mode=2, scale=w["scale"],
                                   window_left=window_left, workspace=ws)
    ro, rq, rkc, rvc, rsl = _expected(orc, w, 2, window_left)
    assert_bits_equal(q, rq, "rotated q")
    assert_bits_equal(kc, rkc, "k cache")
    assert_bits_equal(vc, rvc, "v cache")
    assert torch.equal(sl_new, rsl)
    assert_close(o, ro, 2e-2, "decode step")
    names = [c[0] for c in cpu_ops]
    assert names == ["appendkv", "heuristic", "splitkv", "combine"]
    sk = dict(cpu_ops)["splitkv"]
    assert sk["num_splits"] == 3 and sk["mask_type"] == F.MASK_BOTTOM_RIGHT and sk["window"] == (window_left, 0)
    assert sk["max_seqlen_q"] == w["max_new"]
    # the heuristic is asked about what the block table can address, not about lengths that live on the GPU
    h = dict(cpu_ops)["heuristic"]
    assert h["max_sk"] == w["block_table"].shape[1] * w["k_cache"].shape[1] and h["sq"] == w["max_new"]
    # the caller's lengths are untouched
    assert torch.equal(w["seqlen_k"], gen.workload_appendkv_decode(**dict(seed=7, batch=5, hq=8, hk=2, head_dim=64, min_len=0,
                                                                          max_len=200, max_new=6, page_size=16))["seqlen_k"])


def test_uniform_single_token_step_needs_no_mask(cpu_ops, orc):
    g = torch.Generator().manual_seed(3)
    B, hq, hk, d, page = 4, 4, 2, 64, 16
    lens = [0, 15, 16, 77]
    kv = gen.paged_kv(lens, hk, d, torch.float16, g, page, capacity=[l + 1 for l in lens])
    q = gen.randn((B, 1, hq, d), torch.float16, g)
    knew, vnew = gen.randn((B, 1, hk, d), torch.float16, g), gen.randn((B, 1, hk, d), torch.float16, g)
    kc, vc = kv["k_cache"].clone(), kv["v_cache"].clone()
    o, sl_new = F.fmha_decode_step(q, knew, vnew, kc, vc, kv["seqlen_k"], kv["block_table"], num_splits=2)
    assert torch.equal(sl_new, kv["seqlen_k"] + 1)
    assert [c[0] for c in cpu_ops] == ["appendkv", "splitkv", "combine"]  # an explicit split count skips the heuristic
    sk = dict(cpu_ops)["splitkv"]
    assert sk["mask_type"] == F.MASK_NONE and sk["window"] == (-1, -1) and sk["num_splits"] == 2
    ro = orc.fmha_fwd(q, kc, vc, seqlen_k=(kv["seqlen_k"] + 1).contiguous(), block_table=kv["block_table"])
    assert_close(o, ro, 1e-2, "single-token step")
    assert o.shape == (B, 1, hq, d)


def test_uniform_multi_token_step_is_causal(cpu_ops, orc):
    g = torch.Generator().manual_seed(5)
    B, n, hq, hk, d, page = 3, 4, 4, 4, 64, 16
    lens = [9, 0, 40]
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page, capacity=[l + n for l in lens])
    q = gen.randn((B, n, hq, d), torch.bfloat16, g)
    knew, vnew = gen.randn((B, n, hk, d), torch.bfloat16, g), gen.randn((B, n, hk, d), torch.bfloat16, g)
    kc, vc = kv["k_cache"].clone(), kv["v_cache"].clone()
    o, sl_new = F.fmha_decode_step(q, knew, vnew, kc, vc, kv["seqlen_k"], kv["block_table"], num_splits=3)
    sk = dict(cpu_ops)["splitkv"]
    assert sk["mask_type"] == F.MASK_BOTTOM_RIGHT and sk["window"] == (-1, 0)
    ro = orc.fmha_fwd(q, kc, vc, seqlen_k=(kv["seqlen_k"] + n).contiguous(), block_table=kv["block_table"], mask_type=2,
                      window=(-1, 0))
    assert_close(o, ro, 2e-2, "multi-token step")


def test_workspace_is_reused_and_grows_only_when_needed(cpu_ops, orc):
    ws = F.DecodeWorkspace()
    w = _workload(seed=11)
    args = dict(cu_seqlens_knew=w["cu_seqlens_knew"], max_seqlen_knew=w["max_new"], rotary_cos=w["rotary_cos"],
                rotary_sin=w["rotary_sin"], rope_mode=1, scale=w["scale"], workspace=ws)
    F.fmha_decode_step(w["q"].clone(), w["knew"], w["vnew"], w["k_cache"].clone(), w["v_cache"].clone(), w["seqlen_k"],
                       w["block_table"], **args)
    first = [c[1] for c in cpu_ops if c[0] == "splitkv"][-1]
    ptr_o, ptr_l = first["o_acc"].data_ptr(), first["lse_acc"].data_ptr()
    F.fmha_decode_step(w["q"].clone(), w["knew"], w["vnew"], w["k_cache"].clone(), w["v_cache"].clone(), w["seqlen_k"],
                       w["block_table"], **args)
    second = [c[1] for c in cpu_ops if c[0] == "splitkv"][-1]
    assert second["o_acc"].data_ptr() == ptr_o and second["lse_acc"].data_ptr() == ptr_l
    # a smaller problem fits the same buffers
    small = _workload(seed=12, batch=2, max_new=2)
    F.fmha_decode_step(small["q"].clone(), small["knew"], small["vnew"], small["k_cache"].clone(), small["v_cache"].clone(),
                       small["seqlen_k"], small["block_table"], cu_seqlens_knew=small["cu_seqlens_knew"],
                       max_seqlen_knew=small["max_new"], workspace=ws)
    third = [c[1] for c in cpu_ops if c[0] == "splitkv"][-1]
    assert third["o_acc"].data_ptr() == ptr_o
    total = small["q"].shape[0]
    assert third["o_acc"].shape == (1, 8, 3, total, 64) and third["o_acc"].is_contiguous()


def test_step_argument_errors(cpu_ops):
    w = _workload(seed=13)
    with pytest.raises(ValueError, match="max_seqlen_knew"):
        F.fmha_decode_step(w["q"], w["knew"], w["vnew"], w["k_cache"], w["v_cache"], w["seqlen_k"], w["block_table"],
                           cu_seqlens_knew=w["cu_seqlens_knew"])
    with pytest.raises(ValueError, match=r"\[B, n, Hq, D\]"):
        F.fmha_decode_step(w["q"], w["knew"], w["vnew"], w["k_cache"], w["v_cache"], w["seqlen_k"], w["block_table"])


def test_paged_attention_module_step(cpu_ops, orc):
    from flashck_amd.nn import PagedAttention
    w = _workload(seed=17)
    m = PagedAttention(8, 2, 64, rope_mode=2, scale=w["scale"])
    q, kc, vc = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    o, sl_new = m.decode_step(q, w["knew"], w["vnew"], kc, vc, w["seqlen_k"], w["block_table"],
                              cu_seqlens_knew=w["cu_seqlens_knew"], max_seqlen_knew=w["max_new"],
                              rotary_cos=w["rotary_cos"], rotary_sin=w["rotary_sin"])
    ro, *_ = _expected(orc, w, 2)
    assert_close(o, ro, 2e-2, "module step")
    assert "rope_mode=2" in repr(m)
    with pytest.raises(ValueError, match="module expects"):
        m.decode_step(q[:, :4], w["knew"], w["vnew"], kc, vc, w["seqlen_k"], w["block_table"],
                      cu_seqlens_knew=w["cu_seqlens_knew"], max_seqlen_knew=w["max_new"])


def test_module_constructor_validation():
    from flashck_amd.nn import Attention, PagedAttention
    with pytest.raises(ValueError, match="multiple"):
        Attention(6, 4, 64)
    with pytest.raises(ValueError, match="positive"):
        Attention(8, 0, 64)
    with pytest.raises(ValueError, match="mask_type"):
        Attention(8, 8, 64, mask_type=9)
    with pytest.raises(ValueError, match="rope_mode"):
        PagedAttention(8, 8, 64, rope_mode=5)
    a = Attention(8, 2, 64, 32, window_size=(3, 0), mask_type=2)
    assert a.v_head_dim == 32 and "window_size=(3, 0)" in repr(a)
    with pytest.raises(ValueError, match="seqstart"):
        a(torch.zeros(4, 8, 64), torch.zeros(4, 2, 64), torch.zeros(4, 2, 32), seqstart_q=torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="module expects"):
        a(torch.zeros(1, 4, 8, 32), torch.zeros(1, 4, 2, 64), torch.zeros(1, 4, 2, 32))
