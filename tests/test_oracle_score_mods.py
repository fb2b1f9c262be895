"""Pins the oracle's score modifiers (elementwise bias, ALiBi, logits soft cap) with a library routine (torch SDPA with
an additive attn_mask), the distance diagrams ck_tile publishes for its ALiBi modes, and closed forms - none of which
restates the oracle's own loop."""
import math

import pytest
import torch
import torch.nn.functional as F

from flashck_amd import generators as gen
from test_oracle_attention import flash_mask, sdpa

# The three ALiBi distance patterns for 4 query rows x 6 keys, as drawn in
# ck_tile/ops/fmha/block/block_position_encoding.hpp:19-36 (VERTICAL is added with +slope, the other two with -slope).
DIAGRAM = {
    "vertical": [[0, 1, 2, 3, 4, 5]] * 4,
    "top_left": [[0, 1, 2, 3, 4, 5], [1, 0, 1, 2, 3, 4], [2, 1, 0, 1, 2, 3], [3, 2, 1, 0, 1, 2]],
    "bottom_right": [[2, 1, 0, 1, 2, 3], [3, 2, 1, 0, 1, 2], [4, 3, 2, 1, 0, 1], [5, 4, 3, 2, 1, 0]],
}
# More rows than keys (6 x 4), bottom right: the zero of the last row still sits on the last key.
BOTTOM_RIGHT_6x4 = [[2, 3, 4, 5], [1, 2, 3, 4], [0, 1, 2, 3], [1, 0, 1, 2], [2, 1, 0, 1], [3, 2, 1, 0]]


def additive(mask_bool, extra):
    """float attn_mask for SDPA: `extra` where visible, -inf elsewhere"""
    return torch.where(mask_bool, extra, torch.full_like(extra, float("-inf")))


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
@pytest.mark.parametrize("shape", ["1,1", "1,h", "b,h"])
@pytest.mark.parametrize("mask_type,window", [(0, (-1, -1)), (2, (-1, 0)), (1, (3, 1))])
def test_elementwise_bias_matches_sdpa_additive_mask(orc, dtype, tol, shape, mask_type, window):
    g = torch.Generator().manual_seed(7)
    B, sq, sk, hq, hk, d = 2, 19, 37, 4, 2, 64
    q, k, v = gen.randn((B, sq, hq, d), dtype, g), gen.randn((B, sk, hk, d), dtype, g), gen.randn((B, sk, hk, d), dtype, g)
    bb, bh = (1 if shape[0] == "1" else B), (1 if shape[2] == "1" else hq)
    bias = (gen.randn((bb, bh, sq, sk), dtype, g) * 2).contiguous()
    o, lse = orc.fmha_fwd(q, k, v, return_lse=True, mask_type=mask_type, window=window, bias=bias)
    vis = flash_mask(mask_type, window, sq, sk)
    m = additive(vis[None, None], bias.float().expand(B, hq, sq, sk))
    ref = sdpa(q, k, v, mask=m)
    assert (o.float() - ref).abs().max() <= tol
    s = torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float().repeat_interleave(hq // hk, 2)) / math.sqrt(d) + m
    assert (lse - torch.logsumexp(s, -1)).abs().max() <= 1e-4


def test_elementwise_bias_row_stride_and_group_mode(orc):
    """A bias wider than the key count (row stride > sk), and packed sequences whose rows index the packed query row."""
    g = torch.Generator().manual_seed(8)
    dtype, hq, hk, d = torch.float16, 4, 2, 32
    lens_q, lens_k = [5, 11, 3], [9, 11, 20]
    cuq = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
    q, k, v = gen.randn((sum(lens_q), hq, d), dtype, g), gen.randn((sum(lens_k), hk, d), dtype, g), gen.randn((sum(lens_k), hk, d), dtype, g)
    bias = gen.randn((hq, sum(lens_q), 24), dtype, g).contiguous()   # 24 >= max(lens_k)
    o = orc.fmha_fwd(q, k, v, seqstart_q=cuq, seqstart_k=cuk, bias=bias)
    for b in range(3):
        qs, ks = slice(cuq[b], cuq[b + 1]), slice(cuk[b], cuk[b + 1])
        m = bias[:, qs, :lens_k[b]].float()[None]
        ref = sdpa(q[qs][None], k[ks][None], v[ks][None], mask=m)[0]
        assert (o[qs].float() - ref).abs().max() <= 2e-3


@pytest.mark.parametrize("case", ["no_mask", "top_left_window", "bottom_right_window", "causal_top_left", "causal_bottom_right"])
def test_alibi_matches_the_published_diagrams(orc, case):
    g = torch.Generator().manual_seed(9)
    dtype, sq, sk, hq, hk, d = torch.float16, 4, 6, 4, 2, 32
    q, k, v = gen.randn((2, sq, hq, d), dtype, g), gen.randn((2, sk, hk, d), dtype, g), gen.randn((2, sk, hk, d), dtype, g)
    slopes = torch.tensor([[0.5, 0.25, 0.125, 0.0625], [1.0, 0.3, 0.7, 0.01]], dtype=torch.float32)
    mask_type, window, diagram, sign = {
        "no_mask": (0, (-1, -1), "bottom_right", -1.0),
        "top_left_window": (1, (2, 1), "top_left", -1.0),
        "bottom_right_window": (2, (2, 1), "bottom_right", -1.0),
        "causal_top_left": (1, (-1, 0), "vertical", 1.0),
        "causal_bottom_right": (2, (-1, 0), "vertical", 1.0),
    }[case]
    dist = torch.tensor(DIAGRAM[diagram], dtype=torch.float32)
    vis = flash_mask(mask_type, window, sq, sk)
    for sl in (slopes, slopes[0]):   # [B, Hq] and [Hq] (shared by the batch)
        o, lse = orc.fmha_fwd(q, k, v, return_lse=True, mask_type=mask_type, window=window, alibi_slopes=sl.contiguous())
        per = sl if sl.dim() == 2 else sl[None].expand(2, hq)
        m = additive(vis[None, None].expand(2, hq, sq, sk), sign * per[:, :, None, None] * dist[None, None])
        ref = torch.nan_to_num(sdpa(q, k, v, mask=m), nan=0.0)
        assert (o.float() - ref).abs().max() <= 2e-3
        s = torch.einsum("bqhd,bkhd->bhqk", q.float(), k.float().repeat_interleave(hq // hk, 2)) / math.sqrt(d) + m
        want = torch.logsumexp(s, -1)
        ok = torch.isfinite(want)
        assert (lse[ok] - want[ok]).abs().max() <= 1e-4


def test_alibi_bottom_right_with_more_rows_than_keys(orc):
    g = torch.Generator().manual_seed(10)
    dtype, sq, sk, h, d = torch.float16, 6, 4, 2, 32
    q, k, v = gen.randn((1, sq, h, d), dtype, g), gen.randn((1, sk, h, d), dtype, g), gen.randn((1, sk, h, d), dtype, g)
    sl = torch.tensor([0.4, 0.9], dtype=torch.float32)
    o = orc.fmha_fwd(q, k, v, alibi_slopes=sl)
    m = -sl[None, :, None, None] * torch.tensor(BOTTOM_RIGHT_6x4, dtype=torch.float32)[None, None]
    assert (o.float() - sdpa(q, k, v, mask=m)).abs().max() <= 2e-3


def test_soft_cap_limits_and_closed_form(orc):
    g = torch.Generator().manual_seed(11)
    dtype, sq, sk, hq, hk, d = torch.float16, 7, 29, 4, 2, 64
    q, k, v = gen.randn((2, sq, hq, d), dtype, g) * 3, gen.randn((2, sk, hk, d), dtype, g), gen.randn((2, sk, hk, d), dtype, g)
    plain = orc.fmha_fwd(q, k, v).float()
    # a cap far above every score changes nothing: cap * tanh(x / cap) -> x
    assert (orc.fmha_fwd(q, k, v, logits_soft_cap=1e5).float() - plain).abs().max() <= 2e-3
    # a cap far below every score flattens them to +-cap ~ 0: uniform attention, O = mean of V
    flat = orc.fmha_fwd(q, k, v, logits_soft_cap=1e-4).float()
    mean_v = v.float().mean(1, keepdim=True).repeat_interleave(hq // hk, 2).expand(2, sq, hq, d)
    assert (flat - mean_v).abs().max() <= 2e-3
    # in between: softmax(cap * tanh(scale * qk / cap)) in float64 with library routines
    cap = 2.5
    o, lse = orc.fmha_fwd(q, k, v, return_lse=True, logits_soft_cap=cap)
    s = torch.einsum("bqhd,bkhd->bhqk", q.double(), k.double().repeat_interleave(hq // hk, 2)) / math.sqrt(d)
    s = cap * torch.tanh(s / cap)
    assert s.abs().max() <= cap and s.abs().max() > 0.9 * cap   # the cap really bites on these inputs
    ref = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, -1), v.double().repeat_interleave(hq // hk, 2))
    assert (o.double() - ref).abs().max() <= 2e-3
    assert (lse.double() - torch.logsumexp(s, -1)).abs().max() <= 1e-4
    # the cap is applied before a bias is added: softmax(cap * tanh(.) + bias)
    bias = gen.randn((1, 1, sq, sk), dtype, g).contiguous()
    ob = orc.fmha_fwd(q, k, v, logits_soft_cap=cap, bias=bias)
    refb = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s + bias.double(), -1), v.double().repeat_interleave(hq // hk, 2))
    assert (ob.double() - refb).abs().max() <= 2e-3


def test_split_kv_partials_carry_the_modifiers(orc):
    """Per-split partials with a bias, merged, equal the unsplit result (the splits see the same modified scores)."""
    g = torch.Generator().manual_seed(12)
    dtype, sq, sk, hq, hk, d = torch.bfloat16, 3, 101, 4, 2, 64
    q, k, v = gen.randn((2, sq, hq, d), dtype, g), gen.randn((2, sk, hk, d), dtype, g), gen.randn((2, sk, hk, d), dtype, g)
    sl = torch.tensor([0.5, 0.25, 0.125, 0.0625], dtype=torch.float32)
    for kw in (dict(alibi_slopes=sl), dict(bias=gen.randn((2, hq, sq, sk), dtype, g).contiguous()), dict(logits_soft_cap=1.5)):
        whole = orc.fmha_fwd(q, k, v, mask_type=2, window=(-1, 0), **kw).float()
        o_acc, lse_acc = orc.fmha_splitkv(q, k, v, 4, mask_type=2, window=(-1, 0), **kw)
        merged = orc.splitkv_combine(lse_acc, o_acc, dtype).float()
        assert (merged - whole).abs().max() <= 1.6e-2


def test_fp8_byte_values_match_the_library_type(orc):
    """Every e4m3 byte decodes to what torch.float8_e4m3fn (the OCP format) says it is."""
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    for byte in range(256):
        got = orc.fp8_to_f32(byte)
        assert (math.isnan(got) and math.isnan(ref[byte].item())) or got == ref[byte].item(), byte


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 2e-3), (torch.bfloat16, 1.6e-2)])
def test_fp8_kv_matches_sdpa_on_the_dequantised_cache(orc, dtype, tol):
    g = torch.Generator().manual_seed(13)
    B, sq, sk, hq, hk, d = 2, 3, 77, 4, 2, 64
    kd, vd = 0.05, 0.02
    q = gen.randn((B, sq, hq, d), dtype, g)
    k8 = (gen.randn((B, sk, hk, d), torch.float32, g) / kd).to(torch.float8_e4m3fn)
    v8 = (gen.randn((B, sk, hk, d), torch.float32, g) / vd).to(torch.float8_e4m3fn)
    o, lse = orc.fmha_fwd(q, k8, v8, return_lse=True, mask_type=2, window=(-1, 0), k_descale=kd, v_descale=vd)
    kf, vf = k8.float() * kd, v8.float() * vd
    vis = flash_mask(2, (-1, 0), sq, sk)
    ref = sdpa(q.float(), kf, vf, mask=vis)
    assert (o.float() - ref).abs().max() <= tol
    s = torch.einsum("bqhd,bkhd->bhqk", q.float(), kf.repeat_interleave(hq // hk, 2)) / math.sqrt(d)
    s = s.masked_fill(~vis, float("-inf"))
    assert (lse - torch.logsumexp(s, -1)).abs().max() <= 1e-4
    # the split partials merge to the same result
    o_acc, lse_acc = orc.fmha_splitkv(q, k8, v8, 3, mask_type=2, window=(-1, 0), k_descale=kd, v_descale=vd)
    assert (orc.splitkv_combine(lse_acc, o_acc, dtype).float() - o.float()).abs().max() <= tol
