"""Pins the oracle's attention, split-KV and combine functions with a library routine (torch SDPA), closed forms,
invariants and brute force - none of which restates the oracle's own loop."""
import math

import pytest
import torch
import torch.nn.functional as F

from flashck_amd import generators as gen


def sdpa(q, k, v, mask=None, scale=None):
    """fp32 library reference on [B, s, H, D] tensors with GQA expansion."""
    g = q.shape[2] // k.shape[2]
    qf, kf, vf = (t.float().transpose(1, 2) for t in (q, k, v))
    kf, vf = kf.repeat_interleave(g, 1), vf.repeat_interleave(g, 1)
    return F.scaled_dot_product_attention(qf, kf, vf, attn_mask=mask, scale=scale).transpose(1, 2)


def flash_mask(mask_type, window, sq, sk):
    """The published flash-attention window rule (not the (y, x) coordinates the oracle uses): key j is visible to
    query i iff i + off - left <= j <= i + off + right, off = 0 (top-left) or sk - sq (bottom-right); negative = open."""
    if mask_type == 0:
        return torch.ones(sq, sk, dtype=torch.bool)
    off = 0 if mask_type == 1 else sk - sq
    i = torch.arange(sq)[:, None] + off
    j = torch.arange(sk)[None, :]
    left, right = window
    ok = torch.ones(sq, sk, dtype=torch.bool)
    if left >= 0:
        ok &= j >= i - left
    if right >= 0:
        ok &= j <= i + right
    return ok


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
@pytest.mark.parametrize("hq,hk", [(8, 8), (8, 2), (4, 1)])
def test_matches_sdpa_no_mask(orc, dtype, tol, hq, hk):
    g = torch.Generator().manual_seed(1)
    q, k, v = gen.randn((2, 33, hq, 64), dtype, g), gen.randn((2, 47, hk, 64), dtype, g), gen.randn((2, 47, hk, 64), dtype, g)
    o, lse = orc.fmha_fwd(q, k, v, return_lse=True)
    assert (o.float() - sdpa(q, k, v)).abs().max() <= tol
    s = torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float().repeat_interleave(hq // hk, 2)) / math.sqrt(64)
    assert (lse - torch.logsumexp(s, -1)).abs().max() <= 1e-4


@pytest.mark.parametrize("sq,sk", [(1, 1), (5, 9), (9, 5), (16, 16), (1, 40), (40, 1)])
@pytest.mark.parametrize("mask_type,window", [(1, (-1, 0)), (2, (-1, 0)), (1, (3, 2)), (2, (3, 2)), (2, (0, 0)), (3, (5, 0)),
                                               (1, (-1, -1)), (2, (2, -1))])
def test_masks_match_flash_attention_rule(orc, sq, sk, mask_type, window):
    want = flash_mask(2 if mask_type == 3 else mask_type, window, sq, sk)
    got = torch.tensor([[orc.visible(mask_type, window, sq, sk, i, j) for j in range(sk)] for i in range(sq)])
    assert torch.equal(got, want)
    # and the attention output agrees with SDPA under that boolean mask (rows with no visible key give zeros)
    g = torch.Generator().manual_seed(sq * 100 + sk)
    q, k, v = gen.randn((1, sq, 4, 32), torch.float16, g), gen.randn((1, sk, 2, 32), torch.float16, g), gen.randn((1, sk, 2, 32), torch.float16, g)
    o = orc.fmha_fwd(q, k, v, mask_type=mask_type, window=window).float()
    ref = torch.nan_to_num(sdpa(q, k, v, mask=want), nan=0.0)
    rows = want.any(1)
    assert (o[:, rows] - ref[:, rows]).abs().max() <= 2e-3 if rows.any() else True
    assert (o[:, ~rows] == 0).all()


def test_closed_forms(orc):
    g = torch.Generator().manual_seed(3)
    dt = torch.float16
    q = gen.randn((1, 6, 2, 32), dt, g)
    v = gen.randn((1, 10, 2, 32), dt, g)
    # K = 0: uniform probabilities -> O is the mean of the visible V rows
    o = orc.fmha_fwd(q, torch.zeros(1, 10, 2, 32, dtype=dt), v, mask_type=2, window=(-1, 0)).float()
    for i in range(6):
        n = i + 1 + 4
        assert (o[0, i] - v[0, :n].float().mean(0)).abs().max() <= 2e-3
    # V constant along keys: O equals that constant
    vc = v[:, :1].expand(1, 10, 2, 32).contiguous()
    o = orc.fmha_fwd(q, gen.randn((1, 10, 2, 32), dt, g), vc).float()
    assert (o - vc[:, :1].float()).abs().max() <= 2e-3
    # one key with a dominating logit: O is that key's V row
    k = torch.zeros(1, 10, 2, 32, dtype=dt)
    k[0, 7] = 60.0 * torch.sign(q[0, 0].float()).to(dt)   # q . k[7] = 60 * |q|_1 >> 0 for the query row 0
    o = orc.fmha_fwd(q[:, :1].contiguous(), k, v, scale=1.0).float()
    assert (o[0, 0] - v[0, 7].float()).abs().max() <= 1e-3
    # a single key: O = V
    o = orc.fmha_fwd(q[:, :1].contiguous(), k[:, :1].contiguous(), v[:, :1].contiguous())
    assert torch.equal(o, v[:, :1])


def test_key_permutation_invariance(orc):
    g = torch.Generator().manual_seed(4)
    q, k, v = gen.randn((1, 4, 4, 64), torch.bfloat16, g), gen.randn((1, 50, 2, 64), torch.bfloat16, g), gen.randn((1, 50, 2, 64), torch.bfloat16, g)
    perm = torch.randperm(50, generator=g)
    a = orc.fmha_fwd(q, k, v).float()
    b = orc.fmha_fwd(q, k[:, perm].contiguous(), v[:, perm].contiguous()).float()
    assert (a - b).abs().max() <= 8e-3   # one bf16 ulp at |o| < 1: the summation order changes


@pytest.mark.parametrize("mode", ["group", "block_table", "page_list", "cache_batch_idx"])
def test_addressing_modes_are_bit_identical_to_contiguous(orc, mode):
    """The same logical K/V reached through every addressing mode gives the same bits (the key order is unchanged)."""
    g = torch.Generator().manual_seed(5)
    lens, qn, hq, hk, d, page = [37, 1, 130], [3, 1, 7], 4, 2, 32, 16
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page)
    cuq = torch.tensor([0, 3, 4, 11], dtype=torch.int32)
    q = gen.randn((11, hq, d), torch.bfloat16, g)
    kw = dict(mask_type=2, window=(-1, 0))
    want = torch.cat([orc.fmha_fwd(q[cuq[b]:cuq[b + 1]].unsqueeze(0).contiguous(), kv["k_rows"][b].unsqueeze(0),
                                   kv["v_rows"][b].unsqueeze(0), **kw)[0] for b in range(3)])
    if mode == "group":
        cuk = torch.tensor([0, 37, 38, 168], dtype=torch.int32)
        got = orc.fmha_fwd(q, torch.cat(kv["k_rows"]), torch.cat(kv["v_rows"]), seqstart_q=cuq, seqstart_k=cuk, **kw)
    elif mode == "block_table":
        got = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqstart_q=cuq, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw)
    elif mode == "page_list":
        pages = [-(-l // page) for l in lens]
        indptr = torch.tensor([0] + list(torch.tensor(pages).cumsum(0)), dtype=torch.int32)
        idx = torch.cat([kv["block_table"][b, :pages[b]] for b in range(3)]).contiguous()
        last = torch.tensor([l - (p - 1) * page for l, p in zip(lens, pages)], dtype=torch.int32)
        got = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqstart_q=cuq, kv_indptr=indptr, kv_page_indices=idx,
                           kv_last_page_lens=last, **kw)
    else:
        rows = 140
        kc = torch.full((5, rows, hk, d), float("nan"), dtype=torch.bfloat16)
        vc = torch.full((5, rows, hk, d), float("nan"), dtype=torch.bfloat16)
        idx = torch.tensor([3, 0, 4], dtype=torch.int32)
        for b in range(3):
            kc[idx[b], :lens[b]] = kv["k_rows"][b]
            vc[idx[b], :lens[b]] = kv["v_rows"][b]
        qb = torch.zeros(3, 7, hq, d, dtype=torch.bfloat16)
        # batch mode needs equal query counts: compare sequence 2 only (7 queries) plus the padded others row-wise
        got_b = orc.fmha_fwd(qb.index_copy(0, torch.tensor([2]), q[4:11].unsqueeze(0)), kc, vc, seqlen_k=kv["seqlen_k"],
                             cache_batch_idx=idx, batch=3, **kw)
        assert torch.equal(got_b[2].view(torch.int16), want[4:11].view(torch.int16))
        return
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.isfinite(got.float()).all(), "NaN sentinels of unused page slots leaked into the result"


@pytest.mark.parametrize("d,dv", [(32, 32), (40, 72), (96, 96), (192, 128), (128, 64), (8, 256)])
def test_unequal_and_odd_head_dims_match_sdpa(orc, d, dv):
    # qk_head_dim != v_head_dim and head dims off the 64 / 128 / 256 grid: the library routine takes them as they are
    g = torch.Generator().manual_seed(d + dv)
    q, k, v = gen.randn((2, 9, 4, d), torch.bfloat16, g), gen.randn((2, 31, 2, d), torch.bfloat16, g), gen.randn((2, 31, 2, dv), torch.bfloat16, g)
    o, lse = orc.fmha_fwd(q, k, v, return_lse=True, mask_type=2, window=(-1, 0))
    vis = flash_mask(2, (-1, 0), 9, 31)
    assert o.shape == (2, 9, 4, dv)
    assert (o.float() - sdpa(q, k, v, mask=vis)).abs().max() <= 1.6e-2
    s = torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float().repeat_interleave(2, 2)) / math.sqrt(d)
    assert (lse - torch.logsumexp(s.masked_fill(~vis, float("-inf")), -1)).abs().max() <= 1e-4
    o_acc, lse_acc = orc.fmha_splitkv(q, k, v, 3, mask_type=2, window=(-1, 0))
    assert o_acc.shape == (2, 4, 3, 9, dv)
    comb = orc.splitkv_combine(lse_acc, o_acc, torch.bfloat16)
    assert (comb.float() - o.float()).abs().max() <= 8e-3


@pytest.mark.parametrize("ns", [1, 2, 3, 8, 16])
@pytest.mark.parametrize("mask_type", [0, 2])
def test_splitkv_partials_and_combine(orc, ns, mask_type):
    g = torch.Generator().manual_seed(6 + ns)
    q, k, v = gen.randn((2, 3, 4, 32), torch.bfloat16, g), gen.randn((2, 21, 2, 32), torch.bfloat16, g), gen.randn((2, 21, 2, 32), torch.bfloat16, g)
    kw = dict(mask_type=mask_type, window=(-1, 0) if mask_type else (-1, -1))
    full, lse_full = orc.fmha_fwd(q, k, v, return_lse=True, **kw)
    o_acc, lse_acc = orc.fmha_splitkv(q, k, v, ns, **kw)
    per = -(-21 // ns)
    for s in range(ns):
        k0, k1 = min(per * s, 21), min(per * (s + 1), 21)
        if k1 == k0:
            assert torch.isinf(lse_acc[:, :, s]).all() and (o_acc[:, :, s] == 0).all()   # empty split
            continue
        # each split equals attention restricted to its key range: K/V sliced, mask shifted to the slice
        part_vis = torch.stack([torch.tensor([[orc.visible(mask_type, kw["window"], 3, 21, i, j) for j in range(k0, k1)]
                                              for i in range(3)])])
        ref = torch.nan_to_num(sdpa(q, k[:, k0:k1], v[:, k0:k1], mask=part_vis), nan=0.0)   # [B, sq, H, D]
        got = o_acc[:, :, s].permute(0, 2, 1, 3)
        rows = part_vis[0].any(1)
        assert (got[:, rows] - ref[:, rows]).abs().max() <= 1.6e-2
    # logsumexp over the splits' LSE is the full LSE; combining the partials reproduces the unsplit output
    assert (torch.logsumexp(lse_acc, 2) - lse_full).abs().max() <= 1e-5
    comb, lse_c = orc.splitkv_combine(lse_acc, o_acc, torch.bfloat16, return_lse=True)
    assert (comb.float() - full.float()).abs().max() <= 8e-3
    assert (lse_c - lse_full).abs().max() <= 1e-5
    if ns == 1:
        assert torch.equal(comb.view(torch.int16), o_acc[:, :, 0].permute(0, 2, 1, 3).contiguous().to(torch.bfloat16).view(torch.int16))


def test_combine_closed_form(orc):
    # textbook: O = sum_s softmax_s(lse)_s * O_s; all-masked rows give zeros
    g = torch.Generator().manual_seed(7)
    o_acc = torch.randn(2, 3, 5, 4, 64, generator=g)
    lse = torch.randn(2, 3, 5, 4, generator=g) * 4
    lse[0, 1, 2] = float("-inf")
    lse[1, 0, :, 3] = float("-inf")
    w = torch.nan_to_num(torch.softmax(lse, dim=2), nan=0.0)
    want = (w.unsqueeze(-1) * o_acc).sum(2).permute(0, 2, 1, 3)
    got = orc.splitkv_combine(lse, o_acc, torch.float16).float()
    assert (got - want).abs().max() <= 2e-3
    assert (got[1, 3, 0] == 0).all()
