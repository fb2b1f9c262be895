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


def _pool_bits(t):
    return t.contiguous().view(torch.uint8 if t.dtype == F8 else torch.int16).cpu()


@pytest.mark.parametrize("seed", range(60))
def test_random_appendkv(fmha, orc, seed):
    """Whole pools and the rotated q compared bit for bit: appended rows as the oracle writes them, every other byte
    (NaN fill of unused slots included) untouched."""
    r = random.Random(9000 + seed)
    g = torch.Generator().manual_seed(9000 + seed)
    dtype = r.choice([torch.bfloat16, torch.float16])
    B = r.randint(1, 5)
    hk = r.choice([1, 2, 3, 4])
    hq = hk * r.choice([1, 2, 4])
    fp8 = r.random() < 0.3
    d = r.choice([64, 128, 256] if fp8 else [32, 64, 96, 128, 192, 256])
    dv = d if fp8 or r.random() < 0.7 else r.choice([64, 128])
    page = r.choice([1, 16, 48, 64, 128])
    rope_mode = r.choice([0, 1, 2, 2])
    rotary_dim = r.choice([d, d // 2, 16, d - 16])
    has_mask = r.random() < 0.7
    with_q = r.random() < 0.8
    lens = [r.randint(1, 400) for _ in range(B)]
    new = [r.randint(1, 9) for _ in range(B)]
    uniform = r.random() < 0.3   # [B, n, H, D] inputs without cu_seqlens
    if uniform:
        new = [new[0]] * B
    cap = [l + n for l, n in zip(lens, new)]
    kv = gen.paged_kv(lens, hk, d, dtype, g, page, capacity=cap, dv=dv if dv != d else None)
    total = sum(new)
    cu = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
    q = gen.randn((total, hq, d), dtype, g) if with_q else None
    knew, vnew = gen.randn((total, hk, d), dtype, g), gen.randn((total, hk, dv), dtype, g)
    cos, sin = gen.rotary_tables(max(cap) + 1, rotary_dim, dtype) if rope_mode else (None, None)
    what = (f"seed {seed}: {dtype} B={B} Hq{hq if with_q else 0}/Hk{hk} d=({d},{dv}) P={page} rope={rope_mode}/{rotary_dim} has_mask={has_mask} "
            f"lens={lens} new={new} uniform={uniform} fp8={fp8}")
    print(what, flush=True)
    scales = {}
    if fp8:
        scales = dict(k_descale=r.choice([0.02, 0.05]), v_descale=r.choice([0.01, 0.03]))
        fill = lambda t: torch.full(t.shape, 0x55, dtype=torch.uint8).view(F8)
        kc0, vc0 = fill(kv["k_cache"]), fill(kv["v_cache"])
    else:
        kc0, vc0 = kv["k_cache"], kv["v_cache"]
    dq, kc, vc = dev(q), dev(kc0), dev(vc0)
    if uniform:
        n = new[0]
        shape = lambda t, h, dd: None if t is None else dev(t.view(B, n, h, dd))
        fmha.fmha_fwd_appendkv(shape(q, hq, d), kc, vc, shape(knew, hk, d), shape(vnew, hk, dv), dev(kv["seqlen_k"]), rotary_cos=dev(cos),
                               rotary_sin=dev(sin), rope_mode=rope_mode, has_mask=has_mask, block_table=dev(kv["block_table"]), **scales)
        dq = None  # the view above was copied to the device on its own: compare that copy
        if with_q:
            dq = shape(q, hq, d)
            kc, vc = dev(kc0), dev(vc0)
            fmha.fmha_fwd_appendkv(dq, kc, vc, shape(knew, hk, d), shape(vnew, hk, dv), dev(kv["seqlen_k"]), rotary_cos=dev(cos),
                                   rotary_sin=dev(sin), rope_mode=rope_mode, has_mask=has_mask, block_table=dev(kv["block_table"]), **scales)
    else:
        fmha.fmha_fwd_appendkv(dq, kc, vc, dev(knew), dev(vnew), dev(kv["seqlen_k"]), cu_seqlens_knew=dev(cu), max_seqlen_knew=max(new),
                               rotary_cos=dev(cos), rotary_sin=dev(sin), rope_mode=rope_mode, has_mask=has_mask,
                               block_table=dev(kv["block_table"]), **scales)
    rq = q.clone() if with_q else None
    rkc, rvc = kc0.clone(), vc0.clone()
    orc.appendkv(rq, rkc, rvc, knew, vnew, kv["seqlen_k"], cu, cos=cos, sin=sin, rope_mode=rope_mode, has_mask=has_mask,
                 block_table=kv["block_table"], **scales)
    for name, a, b in (("k_cache", kc, rkc), ("v_cache", vc, rvc)) + ((("q", dq.view(total, hq, d), rq),) if with_q else ()):
        bad = (_pool_bits(a) != _pool_bits(b)).nonzero()
        assert bad.numel() == 0, f"{what}: {name}: {bad.shape[0]} elements differ, first at {bad[0].tolist()}"


@pytest.mark.parametrize("seed", range(60))
def test_random_decode_group_mode_bias_and_cache_rows(fmha, orc, seed):
    """What test_random_decode leaves out: packed queries of ragged length (group mode) over a packed or paged K/V, an
    elementwise bias of every rank, and a batch cache addressed through cache_batch_idx."""
    r = random.Random(13000 + seed)
    g = torch.Generator().manual_seed(13000 + seed)
    dtype = r.choice([torch.bfloat16, torch.float16])
    B = r.randint(1, 4)
    hk = r.choice([1, 2, 4])
    ratio = r.choice([1, 2, 4])
    hq = hk * ratio
    d = r.choice([64, 128, 256])
    ns = r.randint(1, 4)
    mask_type, window = _mask(r)
    layout = r.choice(["group_packed", "group_paged", "batch_rows"])
    lens_k = [r.randint(1, 300) for _ in range(B)]
    common = dict(scale=1.0 / math.sqrt(d), mask_type=mask_type, window=window)
    if layout == "batch_rows":
        sq = r.choice([1, 2, 4])
        rows, slots = max(lens_k) + r.randint(0, 9), B + r.randint(0, 2)
        idx = torch.tensor(r.sample(range(slots), B), dtype=torch.int32)
        k, v = gen.randn((slots, rows, hk, d), dtype, g), gen.randn((slots, rows, hk, d), dtype, g)
        q = gen.randn((B, sq, hq, d), dtype, g)
        sl = torch.tensor(lens_k, dtype=torch.int32)
        bias_rows, group, min_cols = sq, False, rows   # a batch cache: a bias row spans the cache's rows
        dkw = dict(seqlen_k=dev(sl), cache_batch_idx=dev(idx))
        okw = dict(seqlen_k=sl, cache_batch_idx=idx)
        ckw, ockw = {}, {}
    else:
        lens_q = [r.randint(1, 6) for _ in range(B)]
        cq = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
        q = gen.randn((sum(lens_q), hq, d), dtype, g)
        bias_rows, group, min_cols = sum(lens_q), True, max(lens_k)
        if layout == "group_packed":
            ck = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
            k, v = gen.randn((sum(lens_k), hk, d), dtype, g), gen.randn((sum(lens_k), hk, d), dtype, g)
            dkw = dict(cu_seqlens_q=dev(cq), cu_seqlens_k=dev(ck), max_seqlen_q=max(lens_q))
            okw = dict(seqstart_q=cq, seqstart_k=ck)
        else:
            kv = gen.paged_kv(lens_k, hk, d, dtype, g, r.choice([16, 48, 64, 128]))
            k, v = kv["k_cache"], kv["v_cache"]
            dkw = dict(cu_seqlens_q=dev(cq), max_seqlen_q=max(lens_q), seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]))
            okw = dict(seqstart_q=cq, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"])
        ckw, ockw = dict(cu_seqlens_q=dev(cq), max_seqlen_q=max(lens_q)), dict(seqstart_q=cq)
    rank = r.choice([None, 0, 1, 2])
    if rank is not None:
        cols = min_cols + r.choice([0, 0, 5])
        shape = (1 if rank == 0 else hq, bias_rows, cols) if group else (B if rank == 2 else 1, 1 if rank == 0 else hq, bias_rows, cols)
        bias = (gen.randn(shape, dtype, g) * 1.5).contiguous()
        dkw["bias"], okw["bias"] = dev(bias), bias
        if r.random() < 0.3:
            dkw["logits_soft_cap"] = okw["logits_soft_cap"] = 3.0
    what = f"seed {seed}: {layout} {dtype} B={B} Hq{hq}/Hk{hk} d={d} lens_k={lens_k} ns={ns} mask={mask_type}{window} bias rank {rank}"
    print(what, flush=True)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(k), dev(v), ns, **common, **dkw)
    kernel = _lib.load().fck_fmha_last_kernel().decode()
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, dtype, **ckw)
    assert_close(o, orc.fmha_fwd(q, k, v, **common, **okw), ATOL[dtype], what + " [" + kernel + "]")
    ra, rl = orc.fmha_splitkv(q, k, v, ns, **common, **okw)
    assert_lse_close(lse_acc, rl, 2e-3, what + " lse_acc")
    assert_close(o_acc, ra, ATOL[dtype], what + " o_acc")
