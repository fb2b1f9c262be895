"""GPU parity: qk_head_dim != v_head_dim and head dims off the 64 / 128 / 256 grid (padded onto the next kernel size),
through every entry point that takes them, against the CPU oracle."""
import math

import pytest
import torch

from flashck_amd import _lib, generators as gen
from helpers import ATOL, assert_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu

DIMS = [(32, 32), (96, 96), (192, 128), (128, 64), (40, 72), (256, 128), (8, 8), (64, 128), (200, 256)]


def _half(kv):
    """V scaled to |v| < 4: an output row that sees one or two keys is (nearly) a V row, and from magnitude 4 on one
    bf16 ulp (2^-5) is already more than the max-abs tolerance."""
    kv["v_cache"] = kv["v_cache"] * 0.5
    return kv


def _last_kernel():
    return _lib.load().fck_fmha_last_kernel().decode()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,dv", DIMS)
@pytest.mark.parametrize("mask_type,window", [(0, (-1, -1)), (2, (-1, 0))])
def test_dense_forward(fmha, orc, dtype, d, dv, mask_type, window):
    g = torch.Generator().manual_seed(d * 3 + dv)
    q, k, v = gen.randn((2, 150, 4, d), dtype, g), gen.randn((2, 203, 2, d), dtype, g), gen.randn((2, 203, 2, dv), dtype, g) * 0.5
    o = fmha.fmha_fwd(dev(q), dev(k), dev(v), mask_type=mask_type, window=window)
    torch.cuda.synchronize()
    assert "padded_head_dim" in _last_kernel()
    assert o.shape == (2, 150, 4, dv)
    assert_close(o, orc.fmha_fwd(q, k, v, mask_type=mask_type, window=window), ATOL[dtype], "o")


@pytest.mark.parametrize("d,dv", DIMS)
@pytest.mark.parametrize("page,num_splits,sq", [(128, 3, 1), (16, 2, 1), (64, 4, 5), (48, 1, 40)])
def test_paged_splitkv_and_combine(fmha, orc, d, dv, page, num_splits, sq):
    g = torch.Generator().manual_seed(d + 7 * dv + page)
    lens = [sq, 129 + sq, 300, 517]
    kv = _half(gen.paged_kv(lens, 2, d, torch.bfloat16, g, page, dv=dv))
    q = gen.randn((len(lens), sq, 8, d), torch.bfloat16, g)
    kw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=1 / math.sqrt(d), mask_type=2, window=(-1, 0))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), num_splits,
                                           **{k: (dev(v) if isinstance(v, torch.Tensor) else v) for k, v in kw.items()})
    assert "padded_head_dim" in _last_kernel()
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, torch.bfloat16)
    torch.cuda.synchronize()
    assert o_acc.shape == (len(lens), 8, num_splits, sq, dv) and o.shape == (len(lens), sq, 8, dv)
    ro_acc, rlse_acc = orc.fmha_splitkv(q, kv["k_cache"], kv["v_cache"], num_splits, **kw)
    assert_lse_close(lse_acc, rlse_acc, what="lse_acc")
    assert_close(o_acc, ro_acc, ATOL[torch.bfloat16], "o_acc")
    assert_close(o, orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], **kw), ATOL[torch.bfloat16], "o")


@pytest.mark.parametrize("d,dv", [(192, 128), (96, 96), (32, 32), (128, 256)])
@pytest.mark.parametrize("page", [128, 16])
def test_batch_prefill_page_list(fmha, orc, d, dv, page):
    g = torch.Generator().manual_seed(5 + d + dv)
    lens = [1, 130, 300, 77]
    kv = _half(gen.paged_kv(lens, 2, d, torch.bfloat16, g, page, dv=dv))
    cu = torch.zeros(len(lens) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(lens).cumsum(0)
    pages = [-(-l // page) for l in lens]
    indptr = torch.zeros(len(lens) + 1, dtype=torch.int32)
    indptr[1:] = torch.tensor(pages).cumsum(0)
    indices = torch.cat([kv["block_table"][b, :pages[b]] for b in range(len(lens))]).contiguous()
    last = torch.tensor([l - (p - 1) * page for l, p in zip(lens, pages)], dtype=torch.int32)
    q = gen.randn((int(cu[-1]), 4, d), torch.bfloat16, g)
    o = fmha.fmha_batch_prefill(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(cu), dev(indptr), dev(indices), dev(last),
                                max_seqlen_q=max(lens), scale=1 / math.sqrt(d), mask_type=2, window=(-1, 0))
    torch.cuda.synchronize()
    assert "padded_head_dim" in _last_kernel()
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqstart_q=cu, kv_indptr=indptr, kv_page_indices=indices,
                      kv_last_page_lens=last, page_size=page, scale=1 / math.sqrt(d), mask_type=2, window=(-1, 0))
    assert_close(o, ro, ATOL[torch.bfloat16], "o")


def test_block_table_prefill_and_group_mode(fmha, orc):
    d, dv = 192, 128
    g = torch.Generator().manual_seed(23)
    lens, sq = [260, 140], 130
    kv = _half(gen.paged_kv(lens, 2, d, torch.bfloat16, g, 64, dv=dv))
    q = gen.randn((2, sq, 4, d), torch.bfloat16, g)
    kw = dict(scale=1 / math.sqrt(d), mask_type=2, window=(-1, 0))
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), **kw)
    torch.cuda.synchronize()
    assert_close(o, orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw),
                 ATOL[torch.bfloat16], "pagedkv o")
    # packed (group mode) dense forward
    cu = torch.tensor([0, 70, 200], dtype=torch.int32)
    qg, kg, vg = gen.randn((200, 4, d), torch.bfloat16, g), gen.randn((200, 2, d), torch.bfloat16, g), gen.randn((200, 2, dv), torch.bfloat16, g) * 0.5
    og = fmha.fmha_fwd_varlen(dev(qg), dev(kg), dev(vg), dev(cu), dev(cu), max_seqlen_q=130, **kw)
    torch.cuda.synchronize()
    assert_close(og, orc.fmha_fwd(qg, kg, vg, seqstart_q=cu, seqstart_k=cu, **kw), ATOL[torch.bfloat16], "group o")


def test_bias_and_soft_cap_with_padded_dims(fmha, orc):
    d, dv = 96, 160
    g = torch.Generator().manual_seed(29)
    q, k, v = gen.randn((2, 70, 4, d), torch.bfloat16, g), gen.randn((2, 90, 2, d), torch.bfloat16, g), gen.randn((2, 90, 2, dv), torch.bfloat16, g) * 0.5
    bias = gen.randn((2, 4, 70, 90), torch.bfloat16, g)
    slopes = torch.tensor([0.5, 0.25, 0.125, 0.0625], dtype=torch.float32)
    o = fmha.fmha_fwd(dev(q), dev(k), dev(v), bias=dev(bias), logits_soft_cap=20.0)
    torch.cuda.synchronize()
    assert_close(o, orc.fmha_fwd(q, k, v, bias=bias, logits_soft_cap=20.0), ATOL[torch.bfloat16], "bias + cap")
    # decode with ALiBi
    lens = [90, 33]
    kv = _half(gen.paged_kv(lens, 2, d, torch.bfloat16, g, 32, dv=dv))
    qd = gen.randn((2, 1, 4, d), torch.bfloat16, g)
    kw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=1 / math.sqrt(d))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(qd), dev(kv["k_cache"]), dev(kv["v_cache"]), 2, seqlen_k=dev(kv["seqlen_k"]),
                                           block_table=dev(kv["block_table"]), scale=1 / math.sqrt(d), alibi_slopes=dev(slopes))
    od = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, torch.bfloat16)
    torch.cuda.synchronize()
    assert_close(od, orc.fmha_fwd(qd, kv["k_cache"], kv["v_cache"], alibi_slopes=slopes, **kw), ATOL[torch.bfloat16], "alibi decode")


def test_what_padded_dims_do_not_take(fmha):
    g = torch.Generator().manual_seed(31)
    kv = gen.paged_kv([100, 50], 2, 96, torch.bfloat16, g, 32)
    q = dev(gen.randn((2, 1, 4, 96), torch.bfloat16, g))
    args = (q, dev(kv["k_cache"]), dev(kv["v_cache"]))
    kw = dict(seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]))
    with pytest.raises((NotImplementedError, ValueError)):
        fmha.fmha_fwd_splitkv_fused(*args, 2, **kw)
    with pytest.raises((NotImplementedError, ValueError)):
        fmha.fmha_fwd_splitkv(*args, 2, decode_variant=2, **kw)
    with pytest.raises((NotImplementedError, ValueError)):  # head dims are multiples of 8
        fmha.fmha_fwd(dev(gen.randn((1, 8, 2, 36), torch.bfloat16, g)), dev(gen.randn((1, 8, 2, 36), torch.bfloat16, g)),
                      dev(gen.randn((1, 8, 2, 36), torch.bfloat16, g)))
