"""GPU: the all-fp8 roles (Q, K, V, P and O in e4m3 with static scales; FmhaFwdTypeConfig<fp8_t>,
core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171) on the dense, page-list, block-table and split-KV
entry points, against the oracle and against closed forms."""
import math

import pytest
import torch

import helpers
from flashck_amd import _lib, generators as gen
from helpers import assert_fp8_roles_close, dev

pytestmark = pytest.mark.gpu

F8 = torch.float8_e4m3fn
QS, KD, VD = 0.02, 0.025, 0.03  # static scales: stored = value / scale


def _q8(x, s):
    return (x.float() / s).clamp(-448, 448).to(F8)


def _fine(orc, Q, K, V, o_scale=1.0, **kw):
    """The same e4m3 inputs with bf16 roles for Q, P and O (every e4m3 value is a bf16 value): the oracle's fp8-cache mode."""
    return orc.fmha_fwd(Q.float().to(torch.bfloat16), K, V, **kw).float() * o_scale


def _fine_bias(orc, Q, K, V, bias, **kw):
    """_fine with an elementwise bias: the 16-bit roles take the bias in their own type, so it is rounded to bf16 first
    (2^-9 relative: far below an e4m3 step)"""
    return orc.fmha_fwd(Q.float().to(torch.bfloat16), K, V, bias=bias.to(torch.bfloat16), **kw).float()


def _last_kernel():
    return _lib.load().fck_fmha_last_kernel().decode()


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_dense_batch(fmha, orc, d, causal):
    g = torch.Generator().manual_seed(d + causal)
    B, sq, sk, Hq, Hk = 2, 150, 210, 4, 2
    Q = _q8(torch.randn(B, sq, Hq, d, generator=g), QS)
    K = _q8(torch.randn(B, sk, Hk, d, generator=g), KD)
    V = _q8(torch.randn(B, sk, Hk, d, generator=g), VD)
    kw = dict(scale=QS / math.sqrt(d), k_descale=KD, v_descale=VD)
    if causal:
        kw.update(mask_type=2, window=(-1, 0))
    o = fmha.fmha_fwd(dev(Q), dev(K), dev(V), **kw)
    assert o.dtype == F8 and "all_fp8" in _last_kernel()
    assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, **kw), _fine(orc, Q, K, V, **kw), f"dense D={d} causal={causal}")


def test_dense_varlen_alibi_and_soft_cap(fmha, orc):
    g = torch.Generator().manual_seed(9)
    lens_q, lens_k, Hq, Hk, d = [5, 140, 33], [70, 140, 200], 8, 2, 128
    cq = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
    ck = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
    Q = _q8(torch.randn(sum(lens_q), Hq, d, generator=g), QS)
    K = _q8(torch.randn(sum(lens_k), Hk, d, generator=g), KD)
    V = _q8(torch.randn(sum(lens_k), Hk, d, generator=g), VD)
    slopes = torch.rand(Hq, generator=g) * 0.05
    base = dict(scale=QS / math.sqrt(d), k_descale=KD, v_descale=VD, mask_type=2, window=(-1, 0))
    for extra in (dict(alibi_slopes=slopes), dict(logits_soft_cap=3.0)):
        o = fmha.fmha_fwd_varlen(dev(Q), dev(K), dev(V), dev(cq), dev(ck), max(lens_q), **base, **{k: dev(v) for k, v in extra.items()})
        assert "all_fp8" in _last_kernel()
        kw = dict(seqstart_q=cq, seqstart_k=ck, **base, **extra)
        assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, **kw), _fine(orc, Q, K, V, **kw), f"varlen {list(extra)}")


@pytest.mark.parametrize("d,page", [(128, 128), (64, 16), (256, 64)])
def test_batch_prefill_and_pagedkv(fmha, orc, d, page):
    w = gen.workload_varlen_prefill(seed=70 + d + page, batch=3, hq=8, hk=2, head_dim=d, min_len=1, max_len=300, page_size=page,
                                    dtype=torch.bfloat16)
    Q, K, V = _q8(w["q"], QS), _q8(w["k_cache"], KD), _q8(w["v_cache"], VD)
    scale = QS * w["scale"]
    a = [dev(w[k]) for k in ("cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    for o_scale in (1.0, 3.0):
        o = fmha.fmha_batch_prefill(dev(Q), dev(K), dev(V), *a, max_seqlen_q=w["max_seqlen_q"], scale=scale, k_descale=KD, v_descale=VD,
                                    o_scale=o_scale)
        assert o.dtype == F8 and "all_fp8" in _last_kernel()
        kw = dict(seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"], kv_page_indices=w["kv_page_indices"],
                  kv_last_page_lens=w["kv_last_page_lens"], scale=scale, mask_type=2, window=(-1, 0), k_descale=KD, v_descale=VD)
        assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, o_scale=o_scale, **kw), _fine(orc, Q, K, V, o_scale, **kw),
                               f"page list D={d} P={page} o_scale={o_scale}", atol=helpers.FP8_ATOL * o_scale)
    # the same cache through a block table
    B = w["kv_indptr"].numel() - 1
    n_pages = (w["kv_indptr"][1:] - w["kv_indptr"][:-1]).tolist()
    bt = torch.zeros(B, max(n_pages), dtype=torch.int32)
    for b in range(B):
        bt[b, :n_pages[b]] = w["kv_page_indices"][w["kv_indptr"][b]:w["kv_indptr"][b + 1]]
    sl = torch.tensor([(n_pages[b] - 1) * page + int(w["kv_last_page_lens"][b]) for b in range(B)], dtype=torch.int32)
    o = fmha.fmha_fwd_pagedkv(dev(Q), dev(K), dev(V), dev(sl), dev(bt), cu_seqlens_q=dev(w["cu_seqlens_q"]), max_seqlen_q=w["max_seqlen_q"],
                              scale=scale, k_descale=KD, v_descale=VD)
    kw = dict(seqstart_q=w["cu_seqlens_q"], seqlen_k=sl, block_table=bt, scale=scale, mask_type=2, window=(-1, 0), k_descale=KD, v_descale=VD)
    assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, **kw), _fine(orc, Q, K, V, **kw), f"block table D={d} P={page}")


@pytest.mark.parametrize("d,hq,hk,sq", [(128, 32, 8, 1), (64, 8, 2, 1), (256, 4, 2, 1), (128, 4, 2, 5), (128, 16, 2, 1)])
@pytest.mark.parametrize("ns", [1, 3])
def test_splitkv_and_combine(fmha, orc, d, hq, hk, sq, ns):
    g = torch.Generator().manual_seed(11 * d + hq + ns)
    lens = [700, 33, 1500, 260, 1]
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, 64)
    Q = _q8(torch.randn(len(lens), sq, hq, d, generator=g), QS)
    K, V = _q8(kv["k_cache"], KD), _q8(kv["v_cache"], VD)
    kw = dict(scale=QS / math.sqrt(d), k_descale=KD, v_descale=VD, mask_type=2, window=(-1, 0))
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(Q), dev(K), dev(V), ns, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]), **kw)
    assert "all_fp8" in _last_kernel(), _last_kernel()
    assert o_acc.dtype == torch.float32 and lse_acc.dtype == torch.float32
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8)
    assert o.dtype == F8
    okw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw)
    assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, **okw), _fine(orc, Q, K, V, **okw), f"split-KV D={d} Hq={hq}/{hk} sq={sq} ns={ns}")
    # the partial results against those of the 16-bit roles: fp32, apart by the noise of the cast of P only; the LSE
    # never sees that cast
    ra, rl = orc.fmha_splitkv(Q.float().to(torch.bfloat16), K, V, ns, **okw)
    helpers.assert_lse_close(lse_acc, rl, 2e-3, "lse_acc")
    helpers.assert_close(o_acc, ra, helpers.FP8_ATOL, "o_acc")


def _two_key_case(d):
    """Scores (0, -1.25), values (0, 416): the kernel casts P = (1, e^-1.25 = 0.2865) -> (1, 0.28125) and divides by the
    uncast sum 1.2865: 0.28125 * 416 / 1.2865 = 90.9 -> 88 on the e4m3 grid (80, 88, 96).  Without the cast of P the
    result is 0.2865 * 416 / 1.2865 = 92.6 -> 96."""
    q = torch.zeros(1, 1, 1, d)
    q[..., 0] = 1.0
    k = torch.zeros(1, 2, 1, d)
    k[0, 1, 0, 0] = -1.25
    v = torch.zeros(1, 2, 1, d)
    v[0, 1] = 416.0
    return q.to(F8), k.to(F8), v.to(F8)


@pytest.mark.parametrize("d", [64, 128, 256])
def test_p_is_cast_to_e4m3_before_the_second_product(fmha, d):
    q, k, v = (dev(t) for t in _two_key_case(d))
    o = fmha.fmha_fwd(q, k, v, scale=1.0)
    assert torch.all(o.cpu().float() == 88.0), o.cpu().float().unique()
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, k, v, 1, scale=1.0)
    assert abs(o_acc.max().item() - 0.28125 * 416 / (1 + math.exp(-1.25))) < 1e-3, o_acc.max().item()
    assert torch.all(fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8).cpu().float() == 88.0)
    # one key per split: P = 1 in both, the merge weights are fp32 and never cast
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, k, v, 2, scale=1.0)
    assert torch.all(fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8).cpu().float() == 96.0)


def test_output_scale_and_saturation(fmha):
    d = 128
    q = dev(torch.ones(1, 1, 1, d).to(F8))
    k = dev(torch.ones(1, 1, 1, d).to(F8))
    v = torch.full((1, 1, 1, d), 3.0)
    v[..., 1::2] = -3.0
    v = dev(v.to(F8))
    o = fmha.fmha_fwd(q, k, v, scale=0.1, v_descale=0.5, o_scale=16.0).cpu().float()
    assert torch.all(o[..., 0::2] == 24.0) and torch.all(o[..., 1::2] == -24.0)
    o = fmha.fmha_fwd(q, k, v, scale=0.1, v_descale=0.5, o_scale=512.0).cpu().float()
    assert torch.all(o[..., 0::2] == 448.0) and torch.all(o[..., 1::2] == -448.0)
    # the combine saturates as well: a partial result of 3 * 200 = 600
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, k, v, 1, scale=0.1, v_descale=200.0)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8).cpu().float()
    assert torch.all(o[..., 0::2] == 448.0) and torch.all(o[..., 1::2] == -448.0)


def test_what_the_roles_do_not_cover_is_refused(fmha):
    g = torch.Generator().manual_seed(2)
    Q = dev(_q8(torch.randn(1, 4, 2, 128, generator=g), QS))
    K = dev(_q8(torch.randn(1, 40, 2, 128, generator=g), KD))
    with pytest.raises(TypeError):                          # the elementwise bias of these roles is float32
        fmha.fmha_fwd(Q, K, K, bias=dev(torch.zeros(1, 1, 4, 40).to(F8)))
    with pytest.raises(NotImplementedError):                # stored head dims other than 64 / 128 / 256
        fmha.fmha_fwd(dev(_q8(torch.randn(1, 4, 2, 96, generator=g), QS)), dev(_q8(torch.randn(1, 40, 2, 96, generator=g), KD)),
                      dev(_q8(torch.randn(1, 40, 2, 96, generator=g), KD)))
    with pytest.raises(TypeError):                          # fp8 queries over a 16-bit K/V
        fmha.fmha_fwd(Q, dev(K.cpu().float().to(torch.bfloat16)), dev(K.cpu().float().to(torch.bfloat16)))
    kv = gen.paged_kv([100], 2, 128, torch.bfloat16, g, 64)
    Kc, Vc = dev(_q8(kv["k_cache"], KD)), dev(_q8(kv["v_cache"], VD))
    with pytest.raises(NotImplementedError):                # the one-launch entry point has no e4m3 kernels
        fmha.fmha_fwd_splitkv_fused(Q[:, :1], Kc, Vc, 2, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]))


@pytest.mark.parametrize("seed", range(40))
def test_random_problems(fmha, orc, seed):
    """Seeded random problems with e4m3 q / k / v through split-KV + combine and the prefill addressings."""
    import random
    r = random.Random(17000 + seed)
    g = torch.Generator().manual_seed(17000 + seed)
    B = r.randint(1, 4)
    hk = r.choice([1, 2, 4])
    hq = hk * r.choice([1, 2, 4, 8])
    d = r.choice([64, 128, 128, 256])
    page = r.choice([16, 48, 64, 128])
    path = r.choice(["decode", "decode", "page_list", "block_table", "dense_varlen"])
    mask_type, left, right = r.choice([(0, -1, -1), (2, -1, 0), (2, -1, 0), (1, -1, 0), (2, 30, 0), (1, 5, 5)])
    kw = dict(scale=QS / math.sqrt(d), k_descale=KD, v_descale=VD, mask_type=mask_type, window=(left, right))
    extra = {}
    pick = r.random()
    if pick < 0.2:
        extra["alibi_slopes"] = torch.tensor([r.uniform(0.0, 0.05) for _ in range(hq)], dtype=torch.float32)
    elif pick < 0.35:
        extra["logits_soft_cap"] = r.choice([2.0, 20.0])
    dextra = {k: dev(v) for k, v in extra.items()}
    if path == "decode":
        sq, ns = r.choice([1, 1, 2, 4]), r.randint(1, 4)
        lens = [r.randint(1, 700) for _ in range(B)]
        what = f"seed {seed}: decode B={B} Hq{hq}/Hk{hk} sq={sq} d={d} P={page} lens={lens} ns={ns} mask={mask_type}({left},{right}) {sorted(extra)}"
        print(what, flush=True)
        kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, page)
        Q, K, V = _q8(torch.randn(B, sq, hq, d, generator=g), QS), _q8(kv["k_cache"], KD), _q8(kv["v_cache"], VD)
        o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(Q), dev(K), dev(V), ns, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                               **kw, **dextra)
        o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8)
        okw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw, **extra)
    else:
        top = r.choice([20, 140, 260])
        lens_q = [r.randint(1, top) for _ in range(B)]
        lens_k = [n + r.choice([0, 1, 90]) for n in lens_q]
        what = f"seed {seed}: {path} B={B} Hq{hq}/Hk{hk} d={d} P={page} lens_q={lens_q} lens_k={lens_k} mask={mask_type}({left},{right}) {sorted(extra)}"
        print(what, flush=True)
        cq = torch.tensor([0] + list(torch.tensor(lens_q).cumsum(0)), dtype=torch.int32)
        Q = _q8(torch.randn(sum(lens_q), hq, d, generator=g), QS)
        if path == "dense_varlen":
            ck = torch.tensor([0] + list(torch.tensor(lens_k).cumsum(0)), dtype=torch.int32)
            K, V = _q8(torch.randn(sum(lens_k), hk, d, generator=g), KD), _q8(torch.randn(sum(lens_k), hk, d, generator=g), VD)
            o = fmha.fmha_fwd_varlen(dev(Q), dev(K), dev(V), dev(cq), dev(ck), max(lens_q), **kw, **dextra)
            okw = dict(seqstart_q=cq, seqstart_k=ck, **kw, **extra)
        else:
            kv = gen.paged_kv(lens_k, hk, d, torch.bfloat16, g, page)
            K, V = _q8(kv["k_cache"], KD), _q8(kv["v_cache"], VD)
            bt, sl = kv["block_table"], kv["seqlen_k"]
            if path == "page_list":
                n_pages = [(n + page - 1) // page for n in lens_k]
                indptr = torch.tensor([0] + list(torch.tensor(n_pages).cumsum(0)), dtype=torch.int32)
                indices = torch.cat([bt[b, :n_pages[b]] for b in range(B)]).contiguous()
                last = torch.tensor([n - (p - 1) * page for n, p in zip(lens_k, n_pages)], dtype=torch.int32)
                o = fmha.fmha_batch_prefill(dev(Q), dev(K), dev(V), dev(cq), dev(indptr), dev(indices), dev(last), max_seqlen_q=max(lens_q),
                                            **kw, **dextra)
                okw = dict(seqstart_q=cq, kv_indptr=indptr, kv_page_indices=indices, kv_last_page_lens=last, **kw, **extra)
            else:
                o = fmha.fmha_fwd_pagedkv(dev(Q), dev(K), dev(V), dev(sl), dev(bt), cu_seqlens_q=dev(cq), max_seqlen_q=max(lens_q), **kw, **dextra)
                okw = dict(seqstart_q=cq, seqlen_k=sl, block_table=bt, **kw, **extra)
    assert o.dtype == F8 and "all_fp8" in _last_kernel(), _last_kernel()
    assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, **okw), _fine(orc, Q, K, V, **okw), what)


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("rank", [0, 1, 2])
def test_elementwise_bias_is_float32(fmha, orc, d, rank):
    """BiasDataType of these roles is float: every rank, dense forward (batch mode) and paged split-KV + combine."""
    g = torch.Generator().manual_seed(3 * d + rank)
    B, sq, sk, Hq, Hk = 2, 140, 170, 4, 2
    Q = _q8(torch.randn(B, sq, Hq, d, generator=g), QS)
    K = _q8(torch.randn(B, sk, Hk, d, generator=g), KD)
    V = _q8(torch.randn(B, sk, Hk, d, generator=g), VD)
    bias = (torch.randn(B if rank == 2 else 1, 1 if rank == 0 else Hq, sq, sk + 3, generator=g) * 1.5).contiguous()
    kw = dict(scale=QS / math.sqrt(d), k_descale=KD, v_descale=VD, mask_type=2, window=(-1, 0))
    o = fmha.fmha_fwd(dev(Q), dev(K), dev(V), bias=dev(bias), **kw)
    assert "all_fp8" in _last_kernel()
    assert_fp8_roles_close(o, orc.fmha_fwd(Q, K, V, bias=bias, **kw), _fine_bias(orc, Q, K, V, bias, **kw), f"dense D={d} bias rank {rank}")
    # decode: 3 queries per sequence over a paged cache
    lens = [150, 40]
    kv = gen.paged_kv(lens, Hk, d, torch.bfloat16, g, 64)
    Kc, Vc = _q8(kv["k_cache"], KD), _q8(kv["v_cache"], VD)
    Qd = _q8(torch.randn(B, 3, Hq, d, generator=g), QS)
    bd = (torch.randn(B if rank == 2 else 1, 1 if rank == 0 else Hq, 3, max(lens), generator=g) * 1.5).contiguous()
    okw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], **kw)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(Qd), dev(Kc), dev(Vc), 2, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                                           bias=dev(bd), **kw)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, F8)
    assert_fp8_roles_close(o, orc.fmha_fwd(Qd, Kc, Vc, bias=bd, **okw), _fine_bias(orc, Qd, Kc, Vc, bd, **okw), f"decode D={d} bias rank {rank}")
