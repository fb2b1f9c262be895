"""GPU: ALiBi and the logits soft cap on the direct-to-LDS prefill kernels (long query runs, several key tiles, ragged
batches, both page addressings), and the column clamp of a narrow elementwise bias."""
import math

import pytest
import torch

from flashck_amd import _lib, generators as gen
from helpers import ATOL, assert_close, dev

pytestmark = pytest.mark.gpu


def _mods(kind, hq, batch, g):
    if kind == "cap":
        return dict(logits_soft_cap=2.5)
    slopes = (torch.rand(batch, hq, generator=g) * 0.2).float() if kind == "alibi_b" else (torch.rand(hq, generator=g) * 0.2).float()
    kw = dict(alibi_slopes=slopes)
    if kind == "alibi_cap":
        kw["logits_soft_cap"] = 3.0
    return kw


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind", ["cap", "alibi_h", "alibi_b", "alibi_cap"])
@pytest.mark.parametrize("d,page,mask", [(128, 128, (2, (-1, 0))), (64, 64, (2, (100, 0))), (128, 48, (2, (-1, 0))), (256, 64, (2, (-1, 0))),
                                         (256, 128, (1, (-1, 0))), (128, 128, (0, (-1, -1)))])
def test_batch_prefill_with_arithmetic_modifiers(fmha, orc, dtype, kind, d, page, mask):
    """Sequences of 300 / 700 / 129 / 1 tokens: up to 3 row tiles and 11 key tiles per workgroup; page 48 takes the per-row
    lookup variant of the ping-pong kernel."""
    g = torch.Generator().manual_seed(7 + d + page)
    w = gen.workload_varlen_prefill(seed=40 + d + page, batch=4, hq=4, hk=2, head_dim=d, page_size=page, dtype=dtype, lens=[300, 700, 129, 1])
    kw = _mods(kind, 4, 4, g)
    a = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], mask_type=mask[0], window=mask[1],
                                **{k: dev(v) for k, v in kw.items()})
    name = _lib.load().fck_fmha_last_kernel()
    if d == 256:
        assert name == b"prefill_dma_kernel<uniform_page,score_mod>"
    else:
        assert name == (b"prefill_pp_kernel<uniform_page,score_mod>" if page % 64 == 0 else b"prefill_pp_kernel<row_lookup,score_mod>")
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=mask[0],
                      window=mask[1], **kw)
    assert_close(o, ro, ATOL[dtype], f"{kind} on {name.decode()}")


def test_pagedkv_batch_mode_with_alibi_on_the_fast_kernel(fmha, orc):
    g = torch.Generator().manual_seed(23)
    dtype, hq, hk, d, sq = torch.bfloat16, 8, 2, 128, 260
    kv = gen.paged_kv([260, 400], hk, d, dtype, g, 128)
    q = gen.randn((2, sq, hq, d), dtype, g)
    slopes = (torch.rand(2, hq, generator=g) * 0.3).float()
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), mask_type=2,
                              window=(-1, 0), alibi_slopes=dev(slopes))
    assert _lib.load().fck_fmha_last_kernel() == b"prefill_pp_kernel<uniform_page,score_mod>"
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=2, window=(-1, 0),
                      alibi_slopes=slopes)
    assert_close(o, ro, 2e-2, "paged prefill with ALiBi")


@pytest.mark.parametrize("path", ["decode", "prefill"])
def test_narrow_bias_is_clamped_to_its_last_column(fmha, orc, path):
    """A bias with fewer columns than a sequence has keys: reads are clamped to the last column (never out of bounds);
    the oracle gets the same bias widened by repeating that column."""
    g = torch.Generator().manual_seed(29)
    dtype, hq, hk, d = torch.bfloat16, 4, 2, 128
    lens = [90, 200]
    kv = gen.paged_kv(lens, hk, d, dtype, g, 64)
    sq = 1 if path == "decode" else 40
    cols = 120                                    # sequence 1 has 200 keys
    q = gen.randn((2, sq, hq, d), dtype, g)
    bias = gen.randn((2, hq, sq, cols), dtype, g)
    wide = torch.cat([bias, bias[..., -1:].expand(2, hq, sq, 200 - cols)], dim=-1).contiguous()
    args = (dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]))
    if path == "decode":
        o = fmha.fmha_decode_paged(*args, dev(kv["seqlen_k"]), dev(kv["block_table"]), num_splits=2, bias=dev(bias))
    else:
        o = fmha.fmha_fwd_pagedkv(*args, dev(kv["seqlen_k"]), dev(kv["block_table"]), mask_type=2, window=(-1, 0), bias=dev(bias))
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"],
                      mask_type=0 if path == "decode" else 2, window=(-1, -1) if path == "decode" else (-1, 0), bias=wide)
    assert_close(o, ro, 2e-2, f"narrow bias, {path}")


@pytest.mark.parametrize("d,page,sk", [(64, 64, 4400), (128, 128, 8300), (256, 64, 4200)])
@pytest.mark.parametrize("mask", [(2, (-1, 0)), (0, (-1, -1)), (2, (300, 0))])
def test_few_query_rows_over_many_key_tiles(fmha, orc, d, page, sk, mask):
    """200 query rows over up to 130 key tiles of one sequence: the ring buffers wrap many times and the per-workgroup
    cache of first rows is reloaded (it holds 64 tiles per register), at the cost of a short test."""
    g = torch.Generator().manual_seed(d + sk)
    dtype, hq, hk, sq = torch.bfloat16, 2, 1, 200
    kv = gen.paged_kv([sk, 130], hk, d, dtype, g, page)
    q = gen.randn((2, sq, hq, d), dtype, g)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), mask_type=mask[0],
                              window=mask[1])
    name = _lib.load().fck_fmha_last_kernel()
    assert name == (b"prefill_dma_kernel<uniform_page>" if d == 256 else b"prefill_pp_kernel<uniform_page>")
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=mask[0], window=mask[1])
    assert_close(o, ro, 2e-2, f"{name.decode()}, {sk} keys")


@pytest.mark.parametrize("kind", ["cap", "alibi_h", "alibi_b", "alibi_cap", "bias"])
@pytest.mark.parametrize("d,page,fp8", [(128, 128, False), (64, 64, False), (128, 48, False), (128, 128, True)])
def test_head_pair_decode_with_score_modifiers(fmha, orc, kind, d, page, fp8):
    """Score modifiers on the split-KV variant that streams two KV heads per workgroup (forced through the attribute;
    the two heads of a pair have different slopes and bias rows); also over an fp8 cache."""
    g = torch.Generator().manual_seed(3 + d + page)
    dtype, hq, hk, B = torch.bfloat16, 16, 4, 5
    lens = [1, 17, 129, 700, 333]
    kv = gen.paged_kv(lens, hk, d, dtype, g, page)
    q = gen.randn((B, 2, hq, d), dtype, g)        # 2 queries x 4 heads per KV head = 8 packed rows
    if kind == "bias":
        kw = dict(bias=gen.randn((B, hq, 2, 704), dtype, g))
    else:
        kw = _mods(kind, hq, B, g)
    kc, vc, skw = kv["k_cache"], kv["v_cache"], {}
    if fp8:
        skw = dict(k_descale=0.03, v_descale=0.04)
        kc, vc = (kc.float() / 0.03).to(torch.float8_e4m3fn), (vc.float() / 0.04).to(torch.float8_e4m3fn)
    common = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=1 / math.sqrt(d), mask_type=2, window=(-1, 0))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kc), dev(vc), 3, decode_variant=2, **{k: dev(v) for k, v in {**common, **kw}.items()}, **skw)
    name = _lib.load().fck_fmha_last_kernel()
    assert b"head_pairs" in name and b"score_mod" in name and (b"kv_fp8" in name) == fp8
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    ro = orc.fmha_fwd(q, kc, vc, **common, **kw, **skw)
    assert_close(o, ro, 2e-2, f"{kind} on {name.decode()}")
    o1, l1 = fmha.fmha_fwd_splitkv(dev(q), dev(kc), dev(vc), 3, decode_variant=1, **{k: dev(v) for k, v in {**common, **kw}.items()}, **skw)
    assert_close(fmha.fmha_fwd_splitkv_combine(l1, o1, dtype), ro, 2e-2, f"{kind}, one head per workgroup")


@pytest.mark.parametrize("variant", [3, 4])
@pytest.mark.parametrize("d,page", [(128, 128), (64, 64), (128, 32)])
@pytest.mark.parametrize("ns,bound", [(4, 0), (8, 1500), (3, 700), (1, 0)])
def test_splits_of_equal_size_for_a_ragged_batch(fmha, orc, variant, d, page, ns, bound):
    """decode_variant 3 / 4: split s covers keys [s * chunk, (s + 1) * chunk) of every sequence, chunk from the key-count
    bound and num_splits; short sequences leave their last splits empty; a bound below the longest sequence (700 < 1500)
    only moves work into the last split.  Partials against the oracle restricted to those ranges, output against the
    oracle's attention."""
    g = torch.Generator().manual_seed(ns + d)
    dtype, hq, hk = torch.bfloat16, 16, 4
    lens = [1, 31, 32, 33, 500, 1500, 129, 900]
    kv = gen.paged_kv(lens, hk, d, dtype, g, page)
    q = gen.randn((len(lens), 1, hq, d), dtype, g)
    scale = 1 / math.sqrt(d)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), ns, seqlen_k=dev(kv["seqlen_k"]),
                                           block_table=dev(kv["block_table"]), scale=scale, decode_variant=variant, max_seqlen_k=bound)
    name = _lib.load().fck_fmha_last_kernel()
    assert b"equal_chunks" in name and (b"head_pairs" in name) == (variant == 4)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale)
    assert_close(o, ro, 2e-2, name.decode())
    # the partial of (sequence b, split s) is attention over its chunk alone
    capacity = kv["block_table"].shape[1] * page
    limit = bound if 0 < bound < capacity else capacity
    chunk = (-(-limit // ns) + 31) // 32 * 32
    lse = lse_acc.cpu()
    for b, L in enumerate(lens):
        for s in range(ns):
            k0, k1 = min(s * chunk, L), (L if s == ns - 1 else min((s + 1) * chunk, L))
            if k1 <= k0:
                assert torch.isinf(lse[b, :, s]).all() and (lse[b, :, s] < 0).all(), (b, s)
                continue
            sub = orc.fmha_fwd(q[b:b + 1], kv["k_rows"][b][None, k0:k1].contiguous(), kv["v_rows"][b][None, k0:k1].contiguous(), scale=scale)
            assert_close(o_acc[b:b + 1, :, s].cpu().permute(0, 2, 1, 3), sub.float(), 2e-2, f"partial of sequence {b}, split {s}")


def test_equal_size_splits_refusals_and_tuning(fmha, orc, tmp_path, monkeypatch):
    from flashck_amd.utils import flags, tuning
    g = torch.Generator().manual_seed(2)
    kv = gen.paged_kv([100, 900, 40], 4, 128, torch.bfloat16, g, 48)      # pages of 48 keys: not a multiple of 32
    q = gen.randn((3, 1, 16, 128), torch.bfloat16, g)
    with pytest.raises(ValueError, match="splits of equal size"):
        fmha.fmha_fwd_splitkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), 2, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                              decode_variant=3)
    kv = gen.paged_kv([100, 900, 40], 4, 128, torch.bfloat16, g, 128)
    with pytest.raises(ValueError, match="splits of equal size"):
        fmha.fmha_fwd_splitkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), 2, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                              decode_variant=4, logits_soft_cap=2.0)
    # the tuner can record such a variant, and a later automatic call runs it
    cache = tuning.TuningCache(str(tmp_path))
    monkeypatch.setattr(tuning, "default_cache", lambda: cache)
    flags.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "1")
    flags.set_flag_value("FC_TUNING_NUM_REPEATS", "1")
    try:
        args = (dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]))
        rec = fmha.tune_decode_num_splits(*args, max_seqlen_k=900, candidates=(2, 4), variants=(3, 4), cache=cache)
        assert rec["variant"] in (3, 4) and "equal_chunks" in rec["kernel"]
        o = fmha.fmha_decode_paged(*args, max_seqlen_k=900)
        assert b"equal_chunks" in _lib.load().fck_fmha_last_kernel()
    finally:
        flags.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "16")
        flags.set_flag_value("FC_TUNING_NUM_REPEATS", "64")
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"])
    assert_close(o, ro, 2e-2, "automatic call with a recorded equal-size variant")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,dv,page", [(96, 96, 128), (40, 72, 64), (48, 64, 64), (128, 64, 48), (192, 128, 64), (160, 256, 128), (256, 136, 64),
                                       (8, 8, 64)])
@pytest.mark.parametrize("kind", ["none", "alibi_cap"])
def test_padded_head_dims_on_the_fast_kernels(fmha, orc, dtype, d, dv, page, kind):
    """qk_head_dim != v_head_dim and head dims between the instantiated ones, on long query runs: rows keep their stored
    length in memory, the missing columns are zeros in LDS (written once per workgroup) and are never requested."""
    g = torch.Generator().manual_seed(d * 3 + dv)
    hq, hk, lens = 4, 2, [300, 700, 129, 1]
    kv = gen.paged_kv(lens, hk, d, dtype, g, page, dv=dv)
    cu = torch.tensor([0, 300, 1000, 1129, 1130], dtype=torch.int32)
    q = gen.randn((1130, hq, d), dtype, g)
    kw = {} if kind == "none" else _mods(kind, hq, 4, g)
    scale = 1 / math.sqrt(d)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), cu_seqlens_q=dev(cu),
                              max_seqlen_q=700, scale=scale, mask_type=2, window=(-1, 0), **{k: dev(v) for k, v in kw.items()})
    name = _lib.load().fck_fmha_last_kernel()
    big = max(d, dv) > 128
    if big:
        assert name == b"prefill_dma_kernel<uniform_page,padded_head_dim>"
    else:
        assert name == (b"prefill_pp_kernel<uniform_page,padded_head_dim>" if page % 64 == 0 else b"prefill_pp_kernel<row_lookup,padded_head_dim>")
    assert tuple(o.shape) == (1130, hq, dv)
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqstart_q=cu, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale,
                      mask_type=2, window=(-1, 0), **kw)
    assert_close(o, ro, ATOL[dtype], f"({d}, {dv}) on {name.decode()}")


def test_padded_head_dims_dense_batch_mode(fmha, orc):
    g = torch.Generator().manual_seed(41)
    for d, dv in ((192, 128), (80, 80)):
        q, k, v = gen.randn((2, 200, 4, d), torch.bfloat16, g), gen.randn((2, 260, 2, d), torch.bfloat16, g), gen.randn((2, 260, 2, dv), torch.bfloat16, g)
        o = fmha.fmha_fwd(dev(q), dev(k), dev(v), mask_type=2, window=(-1, 0))
        assert b"padded_head_dim" in _lib.load().fck_fmha_last_kernel() and b"prefill_kernel" not in _lib.load().fck_fmha_last_kernel()
        ro = orc.fmha_fwd(q, k, v, mask_type=2, window=(-1, 0))
        assert_close(o, ro, 2e-2, f"dense ({d}, {dv})")
