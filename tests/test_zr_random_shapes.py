"""GPU: seeded random problems through the decode and prefill entry points against the oracle.  The hand-picked cases of
the other files sit on the edges someone thought of; these walk the product of head ratios, ragged key counts, page
sizes, head dims (on and off the 64 / 128 / 256 grid, qk != v), masks and windows, score modifiers, fp8 caches, split
counts and kernel variants.  Every case is reproducible from its seed alone."""
import math
import random

import pytest
import torch

from flashck_amd import _lib, generators as gen
from helpers import ATOL, assert_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu

F8 = torch.float8_e4m3fn


def _mask(r, allow_generic=True):
    """(mask_type, window): no mask, or a top-left / bottom-right (/ generic) window that is causal, sliding or two-sided."""
    kind = r.choice([0, 1, 2, 2, 3] if allow_generic else [0, 1, 2, 2])
    if kind == 0:
        return 0, (-1, -1)
    left = r.choice([-1, -1, 0, 3, 40])
    right = r.choice([0, 0, 0, 5]) if left >= 0 else r.choice([0, 0, 7])
    return kind, (left, right)


def _head_dims(r, allow_pad):
    if allow_pad and r.random() < 0.3:
        return r.choice([(40, 40), (72, 64), (96, 128), (192, 128), (128, 64), (8, 16), (136, 256)])
    d = r.choice([64, 128, 128, 256])
    return d, d


def _mods(r, hq, batch, mask_type):
    """ALiBi slopes (per head or per sequence and head), a soft cap, or nothing"""
    kw, okw = {}, {}
    pick = r.random()
    if pick < 0.25 and mask_type != 3:
        s = torch.tensor([r.uniform(0.0, 0.08) for _ in range(hq * batch)], dtype=torch.float32)
        s = s.view(batch, hq) if r.random() < 0.5 else s[:hq].contiguous()
        kw["alibi_slopes"], okw["alibi_slopes"] = dev(s), s
    elif pick < 0.45:
        kw["logits_soft_cap"] = okw["logits_soft_cap"] = r.choice([1.5, 4.0, 30.0])
    return kw, okw


def _quantise(kv, r):
    kd, vd = r.choice([0.02, 0.03]), r.choice([0.02, 0.05])
    k8 = (kv["k_cache"].float() / kd).clamp(-448, 448).to(F8)
    v8 = (kv["v_cache"].float() / vd).clamp(-448, 448).to(F8)
    return k8, v8, dict(k_descale=kd, v_descale=vd)


@pytest.mark.parametrize("seed", range(120))
def test_random_decode(fmha, orc, seed):
    r = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(1000 + seed)
    dtype = r.choice([torch.bfloat16, torch.float16])
    B = r.randint(1, 5)
    hk = r.choice([1, 2, 3, 4, 8])
    ratio = r.choice([1, 2, 4, 8, 16])
    hq = hk * ratio
    sq = r.choice([1, 1, 1, 2, 3, 5])
    fp8 = r.random() < 0.25
    d, dv = _head_dims(r, allow_pad=not fp8)
    page = r.choice([1, 16, 32, 48, 64, 128])
    top = r.choice([40, 300, 900])
    lens = [r.randint(1, top) for _ in range(B)]
    ns = r.randint(1, 6)
    mask_type, window = _mask(r)
    kv = gen.paged_kv(lens, hk, d, dtype, g, page, dv=dv if dv != d else None)
    q = gen.randn((B, sq, hq, d), dtype, g)
    kw, okw = _mods(r, hq, B, mask_type)
    kc, vc = kv["k_cache"], kv["v_cache"]
    if fp8:
        kc, vc, scales = _quantise(kv, r)
        kw.update(scales)
        okw.update(scales)
    plain = not kw and d == dv and d in (64, 128, 256)
    variant = 0
    if plain and page % 32 == 0 and sq * ratio <= 16 and r.random() < 0.8:
        variant = r.choice([1, 2, 3, 4]) if hk % 2 == 0 and d <= 128 else r.choice([1, 3] if d <= 128 else [1])
    what = (f"seed {seed}: {dtype} B={B} Hq{hq}/Hk{hk} sq={sq} d=({d},{dv}) P={page} lens={lens} ns={ns} mask={mask_type}{window} "
            f"fp8={fp8} variant={variant} {sorted(okw)}")
    print(what, flush=True)
    common = dict(scale=1.0 / math.sqrt(d), mask_type=mask_type, window=window)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kc), dev(vc), ns, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                           decode_variant=variant, max_seqlen_k=max(lens) if variant >= 3 else 0, **common, **kw)
    kernel = _lib.load().fck_fmha_last_kernel().decode()
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype)
    ro, rlse = orc.fmha_fwd(q, kc, vc, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], return_lse=True, **common, **okw)
    assert_close(o, ro, ATOL[dtype], what + " [" + kernel + "]")
    if variant < 3:   # equal-size splits cut the keys elsewhere than the oracle's equal parts: only the merged result compares
        ra, rl = orc.fmha_splitkv(q, kc, vc, ns, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **common, **okw)
        assert_lse_close(lse_acc, rl, 2e-3, what + " lse_acc")
        assert_close(o_acc, ra, ATOL[dtype], what + " o_acc")


@pytest.mark.parametrize("seed", range(120))
def test_random_prefill(fmha, orc, seed):
    r = random.Random(5000 + seed)
    g = torch.Generator().manual_seed(5000 + seed)
    dtype = r.choice([torch.bfloat16, torch.float16])
    B = r.randint(1, 4)
    hk = r.choice([1, 2, 4])
    hq = hk * r.choice([1, 2, 4])
    fp8 = r.random() < 0.2
    d, dv = _head_dims(r, allow_pad=not fp8)
    page = r.choice([16, 64, 64, 128, 48])
    path = r.choice(["page_list", "block_table", "block_table_batch", "dense_varlen"])
    # query runs on both sides of the 128-row switch between the kernels, key counts at least as long
    top = r.choice([20, 140, 300])
    lens_q = [r.randint(1, top) for _ in range(B)]
    if path == "block_table_batch":
        lens_q = [lens_q[0]] * B
    lens_k = [n + r.choice([0, 0, 1, 70, 200]) for n in lens_q]
    mask_type, window = _mask(r)
    cq = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
    q = gen.randn((sum(lens_q), hq, d), dtype, g)
    kw, okw = _mods(r, hq, B, mask_type)
    common = dict(scale=1.0 / math.sqrt(d), mask_type=mask_type, window=window)
    what = (f"seed {seed}: {path} {dtype} B={B} Hq{hq}/Hk{hk} d=({d},{dv}) P={page} lens_q={lens_q} lens_k={lens_k} mask={mask_type}{window} "
            f"fp8={fp8} {sorted(okw)}")
    print(what, flush=True)
    if path == "dense_varlen":
        ck = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
        k = gen.randn((sum(lens_k), hk, d), dtype, g)
        v = gen.randn((sum(lens_k), hk, dv), dtype, g)
        o = fmha.fmha_fwd_varlen(dev(q), dev(k), dev(v), dev(cq), dev(ck), max(lens_q), **common, **kw)
        ro = orc.fmha_fwd(q, k, v, seqstart_q=cq, seqstart_k=ck, **common, **okw)
    else:
        kv = gen.paged_kv(lens_k, hk, d, dtype, g, page, dv=dv if dv != d else None)
        kc, vc = kv["k_cache"], kv["v_cache"]
        if fp8:
            kc, vc, scales = _quantise(kv, r)
            kw.update(scales)
            okw.update(scales)
        bt, sl = kv["block_table"], kv["seqlen_k"]
        if path == "page_list":
            n_pages = [(n + page - 1) // page for n in lens_k]
            indptr = torch.tensor([0] + list(torch.tensor(n_pages).cumsum(0)), dtype=torch.int32)
            indices = torch.cat([bt[b, :n_pages[b]] for b in range(B)]).contiguous()
            last = torch.tensor([n - (p - 1) * page for n, p in zip(lens_k, n_pages)], dtype=torch.int32)
            o = fmha.fmha_batch_prefill(dev(q), dev(kc), dev(vc), dev(cq), dev(indptr), dev(indices), dev(last), max_seqlen_q=max(lens_q),
                                        **common, **kw)
            ro = orc.fmha_fwd(q, kc, vc, seqstart_q=cq, kv_indptr=indptr, kv_page_indices=indices, kv_last_page_lens=last, **common, **okw)
        elif path == "block_table":
            o = fmha.fmha_fwd_pagedkv(dev(q), dev(kc), dev(vc), dev(sl), dev(bt), cu_seqlens_q=dev(cq), max_seqlen_q=max(lens_q), **common, **kw)
            ro = orc.fmha_fwd(q, kc, vc, seqstart_q=cq, seqlen_k=sl, block_table=bt, **common, **okw)
        else:
            qb = q.view(B, lens_q[0], hq, d)
            o = fmha.fmha_fwd_pagedkv(dev(qb), dev(kc), dev(vc), dev(sl), dev(bt), **common, **kw)
            ro = orc.fmha_fwd(qb, kc, vc, seqlen_k=sl, block_table=bt, **common, **okw)
    kernel = _lib.load().fck_fmha_last_kernel().decode()
    assert_close(o, ro, ATOL[dtype], what + " [" + kernel + "]")
