"""GPU parity: appendKV (rotary embedding + paged-cache write) must be bit-exact against the CPU oracle."""
import math

import pytest
import torch

from flashck_amd import generators as gen
from helpers import assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu


def _append_both(fmha, orc, w, rope_mode, has_mask=True, with_q=True):
    """Runs the HIP kernel and the oracle on copies of the same inputs; returns both result sets."""
    q_ref = w["q"].clone() if with_q else None
    kc_ref, vc_ref = w["k_cache"].clone(), w["v_cache"].clone()
    cos, sin = (w["rotary_cos"], w["rotary_sin"]) if rope_mode else (None, None)
    orc.appendkv(q_ref, kc_ref, vc_ref, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos, sin,
                 rope_mode=rope_mode, has_mask=has_mask, block_table=w["block_table"])
    q = dev(w["q"].clone()) if with_q else None
    kc, vc = dev(w["k_cache"].clone()), dev(w["v_cache"].clone())
    fmha.fmha_fwd_appendkv(q, kc, vc, dev(w["knew"]), dev(w["vnew"]), dev(w["seqlen_k"]),
                           cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=w["max_new"],
                           rotary_cos=dev(cos), rotary_sin=dev(sin), rope_mode=rope_mode, has_mask=has_mask,
                           block_table=dev(w["block_table"]))
    torch.cuda.synchronize()
    return (q, kc, vc), (q_ref, kc_ref, vc_ref)


def _check(got, ref):
    # the whole pool is compared: rows outside the appended range (NaN-filled or older tokens) must be untouched
    assert_bits_equal(got[1], ref[1], "k_cache")
    assert_bits_equal(got[2], ref[2], "v_cache")
    if ref[0] is not None:
        assert_bits_equal(got[0], ref[0], "q (rotated in place)")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rope_mode", [0, 1, 2])
@pytest.mark.parametrize("page", [16, 128])
def test_appendkv_small(fmha, orc, dtype, rope_mode, page):
    w = gen.workload_appendkv_decode(seed=100 + rope_mode + page, batch=6, hq=8, hk=2, head_dim=64, min_len=0, max_len=300,
                                     max_new=16, page_size=page, dtype=dtype)
    _check(*_append_both(fmha, orc, w, rope_mode))


def test_appendkv_page_straddle_and_page_start(fmha, orc):
    # existing lengths that put the new tokens across a page border and exactly at a page start
    g = torch.Generator().manual_seed(21)
    page, hk, hq, d = 128, 8, 32, 128
    lens, new = [120, 128, 255, 0, 127], [16, 5, 2, 9, 1]
    cap = [l + n for l, n in zip(lens, new)]
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page, capacity=cap)
    cu = torch.zeros(len(new) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(new).cumsum(0)
    cos, sin = gen.rotary_tables(max(cap) + 1, d, torch.bfloat16)
    kv.update(q=gen.randn((sum(new), hq, d), torch.bfloat16, g), knew=gen.randn((sum(new), hk, d), torch.bfloat16, g),
              vnew=gen.randn((sum(new), hk, d), torch.bfloat16, g), cu_seqlens_knew=cu, rotary_cos=cos, rotary_sin=sin,
              max_new=max(new))
    for has_mask in (True, False):
        _check(*_append_both(fmha, orc, kv, 2, has_mask=has_mask))


def test_appendkv_partial_rotary_dim(fmha, orc):
    w = gen.workload_appendkv_decode(seed=31, batch=4, hq=4, hk=4, head_dim=128, min_len=5, max_len=200, max_new=7,
                                     page_size=64)
    cos, sin = gen.rotary_tables(w["rotary_cos"].shape[0], 64, torch.bfloat16)  # rotary_dim 64 < head_dim 128
    w["rotary_cos"], w["rotary_sin"] = cos, sin
    for mode in (1, 2):
        got, ref = _append_both(fmha, orc, w, mode)
        _check(got, ref)
    # the tail beyond rotary_dim is copied verbatim
    n0 = 0
    L0 = int(w["seqlen_k"][0])
    page = int(w["block_table"][0, L0 // 64])
    row = got[1][page, L0 % 64, 0].cpu()
    assert_bits_equal(row[64:], w["knew"][n0, 0, 64:], "unrotated tail")


def test_appendkv_position_zero_is_identity(fmha, orc):
    # cos(0) = 1, sin(0) = 0: a token appended at position 0 is stored unchanged
    g = torch.Generator().manual_seed(4)
    kv = gen.paged_kv([0], 2, 64, torch.float16, g, 16, capacity=[1])
    cos, sin = gen.rotary_tables(4, 64, torch.float16)
    knew, vnew = gen.randn((1, 2, 64), torch.float16, g), gen.randn((1, 2, 64), torch.float16, g)
    kc, vc = dev(kv["k_cache"].clone()), dev(kv["v_cache"].clone())
    fmha.fmha_fwd_appendkv(None, kc, vc, dev(knew), dev(vnew), dev(kv["seqlen_k"]), cu_seqlens_knew=dev(torch.tensor([0, 1], dtype=torch.int32)),
                           max_seqlen_knew=1, rotary_cos=dev(cos), rotary_sin=dev(sin), rope_mode=2, block_table=dev(kv["block_table"]))
    page = int(kv["block_table"][0, 0])
    assert_bits_equal(kc[page, 0], knew[0], "k at position 0")
    assert_bits_equal(vc[page, 0], vnew[0], "v at position 0")


def test_appendkv_uniform_batch_form(fmha, orc):
    # ck_tile's form: the same number of new tokens for every sequence, knew [B, n, Hk, D], non-paged cache
    g = torch.Generator().manual_seed(8)
    B, n, hk, hq, d, rows = 3, 4, 2, 4, 64, 40
    kc = gen.randn((5, rows, hk, d), torch.bfloat16, g)
    vc = gen.randn((5, rows, hk, d), torch.bfloat16, g)
    knew, vnew = gen.randn((B, n, hk, d), torch.bfloat16, g), gen.randn((B, n, hk, d), torch.bfloat16, g)
    q = gen.randn((B, n, hq, d), torch.bfloat16, g)
    sl = torch.tensor([0, 36, 17], dtype=torch.int32)
    idx = torch.tensor([3, 1, 4], dtype=torch.int32)
    cos, sin = gen.rotary_tables(rows + 1, d, torch.bfloat16)
    cu = torch.arange(0, (B + 1) * n, n, dtype=torch.int32)
    q_ref, kc_ref, vc_ref = q.clone().view(B * n, hq, d), kc.clone(), vc.clone()
    orc.appendkv(q_ref, kc_ref, vc_ref, knew.view(B * n, hk, d), vnew.view(B * n, hk, d), sl, cu, cos, sin, rope_mode=1,
                 has_mask=True, cache_batch_idx=idx)
    qd, kcd, vcd = dev(q.clone()), dev(kc.clone()), dev(vc.clone())
    fmha.fmha_fwd_appendkv(qd, kcd, vcd, dev(knew), dev(vnew), dev(sl), rotary_cos=dev(cos), rotary_sin=dev(sin),
                           rope_mode=1, cache_batch_idx=dev(idx))
    assert_bits_equal(kcd, kc_ref, "k_cache")
    assert_bits_equal(vcd, vc_ref, "v_cache")
    assert_bits_equal(qd.view(B * n, hq, d), q_ref, "q")


def test_workload4_full_append_then_decode(fmha, orc):
    w = gen.workload_appendkv_decode()
    got, ref = _append_both(fmha, orc, w, 2)
    _check(got, ref)
    # decode the new queries (bottom-right causal) over the L_b + n_b keys now in the cache
    q, kc, vc = got
    sl_new = (w["seqlen_k"] + torch.tensor(w["new"], dtype=torch.int32)).contiguous()
    cu = w["cu_seqlens_knew"]
    ns = 4
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, kc, vc, ns, seqlen_k=dev(sl_new), block_table=dev(w["block_table"]),
                                           cu_seqlens_q=dev(cu), max_seqlen_q=w["max_new"], scale=w["scale"], mask_type=2,
                                           window=(-1, 0))
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, cu_seqlens_q=dev(cu), max_seqlen_q=w["max_new"])
    ro = orc.fmha_fwd(ref[0], ref[1], ref[2], seqstart_q=cu, seqlen_k=sl_new, block_table=w["block_table"], scale=w["scale"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "decode after append")
