"""GPU parity: dense / varlen / paged prefill kernels against the CPU oracle (called through the C ABI)."""
import math

import pytest
import torch

from flashck_amd import generators as gen
from helpers import ATOL, assert_close, dev

pytestmark = pytest.mark.gpu


def test_workload1_dense_fp16(fmha, orc):
    w = gen.workload_dense_fp16()
    o = fmha.fmha_fwd(dev(w["q"]), dev(w["k"]), dev(w["v"]), scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k"], w["v"], scale=w["scale"])
    assert_close(o, ro, 1e-2, "dense fp16")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sq,sk,hq,hk,d", [(1, 1, 2, 2, 64), (5, 9, 4, 2, 64), (130, 70, 4, 4, 128), (257, 300, 8, 2, 128),
                                           (64, 64, 2, 1, 256), (200, 333, 4, 2, 256)])
@pytest.mark.parametrize("mask", [(0, (-1, -1)), (1, (-1, 0)), (2, (-1, 0)), (2, (30, 0)), (1, (10, 5))])
def test_dense_batch_mode(fmha, orc, dtype, sq, sk, hq, hk, d, mask):
    g = torch.Generator().manual_seed(sq * 7 + sk + d)
    q = gen.randn((2, sq, hq, d), dtype, g)
    k = gen.randn((2, sk, hk, d), dtype, g)
    v = gen.randn((2, sk, hk, d), dtype, g)
    mt, win = mask
    o = fmha.fmha_fwd(dev(q), dev(k), dev(v), mask_type=mt, window=win)
    ro = orc.fmha_fwd(q, k, v, mask_type=mt, window=win)
    assert_close(o, ro, ATOL[dtype], "dense")


def test_dense_group_mode(fmha, orc):
    g = torch.Generator().manual_seed(17)
    ql, kl = [3, 140, 1, 64], [10, 140, 7, 200]
    cuq = torch.tensor([0] + list(torch.tensor(ql).cumsum(0)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(torch.tensor(kl).cumsum(0)), dtype=torch.int32)
    q = gen.randn((sum(ql), 8, 128), torch.bfloat16, g)
    k = gen.randn((sum(kl), 2, 128), torch.bfloat16, g)
    v = gen.randn((sum(kl), 2, 128), torch.bfloat16, g)
    o = fmha.fmha_fwd_varlen(dev(q), dev(k), dev(v), dev(cuq), dev(cuk), max(ql), mask_type=2, window=(-1, 0))
    ro = orc.fmha_fwd(q, k, v, seqstart_q=cuq, seqstart_k=cuk, mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "group mode")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("page", [16, 64, 128])
def test_batch_prefill_small(fmha, orc, dtype, d, page):
    w = gen.workload_varlen_prefill(seed=50 + d + page, batch=5, hq=4, hk=2, head_dim=d, min_len=1, max_len=400,
                                    page_size=page, dtype=dtype)
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), dev(w["cu_seqlens_q"]), dev(w["kv_indptr"]),
                                dev(w["kv_page_indices"]), dev(w["kv_last_page_lens"]), max_seqlen_q=w["max_seqlen_q"],
                                scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, ATOL[dtype], "batch prefill")


def test_pagedkv_prefill_chunked(fmha, orc):
    # chunked prefill: sq new queries attend to sk >= sq cached keys through a block table (bottom-right causal)
    g = torch.Generator().manual_seed(23)
    lens, qn = [300, 64, 700], [100, 64, 1]
    kv = gen.paged_kv(lens, 2, 128, torch.bfloat16, g, 128)
    cu = torch.tensor([0] + list(torch.tensor(qn).cumsum(0)), dtype=torch.int32)
    q = gen.randn((sum(qn), 8, 128), torch.bfloat16, g)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]),
                              cu_seqlens_q=dev(cu), max_seqlen_q=max(qn))
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqstart_q=cu, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "paged prefill")


def test_dense_group_mode_padded_keys(fmha, orc):
    """Packed K/V whose slots hold padding behind the keys: seqlen_k gives the logical key counts
    (ck_tile/ops/fmha/kernel/fmha_fwd_splitkv_kernel.hpp:648-650); the padding rows are NaN and must not be read."""
    g = torch.Generator().manual_seed(19)
    ql, kl, pad = [5, 200, 64], [9, 300, 64], [7, 20, 0]
    cuq = torch.tensor([0] + list(torch.tensor(ql).cumsum(0)), dtype=torch.int32)
    slots = [k + p for k, p in zip(kl, pad)]
    cuk = torch.tensor([0] + list(torch.tensor(slots).cumsum(0)), dtype=torch.int32)
    sl = torch.tensor(kl, dtype=torch.int32)
    q = gen.randn((sum(ql), 8, 128), torch.bfloat16, g)
    k = torch.full((sum(slots), 2, 128), float("nan"), dtype=torch.bfloat16)
    v = torch.full((sum(slots), 2, 128), float("nan"), dtype=torch.bfloat16)
    kc, vc = [], []
    for b, n in enumerate(kl):
        kb, vb = gen.randn((n, 2, 128), torch.bfloat16, g), gen.randn((n, 2, 128), torch.bfloat16, g)
        k[cuk[b]:cuk[b] + n], v[cuk[b]:cuk[b] + n] = kb, vb
        kc.append(kb)
        vc.append(vb)
    o = fmha.fmha_fwd_varlen(dev(q), dev(k), dev(v), dev(cuq), dev(cuk), max(ql), mask_type=2, window=(-1, 0), seqlen_k=dev(sl))
    # oracle on the compacted keys (no padding, no seqlen_k): an independent statement of the same problem
    cuc = torch.tensor([0] + list(torch.tensor(kl).cumsum(0)), dtype=torch.int32)
    ro = orc.fmha_fwd(q, torch.cat(kc), torch.cat(vc), seqstart_q=cuq, seqstart_k=cuc, mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "padded group mode")
    # split-KV group mode with the same padded layout
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(k), dev(v), 3, seqlen_k=dev(sl), cu_seqlens_q=dev(cuq), cu_seqlens_k=dev(cuk),
                                           max_seqlen_q=max(ql), mask_type=2, window=(-1, 0))
    o2 = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, cu_seqlens_q=dev(cuq), max_seqlen_q=max(ql))
    assert_close(o2, ro, 2e-2, "padded group mode, split-KV")


@pytest.mark.parametrize("sq,d", [(1, 128), (40, 128), (300, 64), (130, 256)])
def test_pagedkv_prefill_batch_mode(fmha, orc, sq, d):
    """Block-table prefill in batch mode (seqstart_q == NULL): every sequence has sq queries over its own key count."""
    g = torch.Generator().manual_seed(29 + sq)
    lens = [max(sq, 333), sq + 1, 1000]
    kv = gen.paged_kv(lens, 2, d, torch.bfloat16, g, 128)
    q = gen.randn((len(lens), sq, 4, d), torch.bfloat16, g)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]))
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=2,
                      window=(-1, 0))
    assert_close(o, ro, 2e-2, "paged prefill, batch mode")


def test_prefill_large_pool_short_sequences(fmha, orc):
    """A serving-size pool (more than 262,144 token slots) with short prompts must still take the kernel variant that
    resolves a tile's page once (not the per-row lookup variant), and stay exact."""
    from flashck_amd import _lib
    g = torch.Generator().manual_seed(37)
    lens = [300, 129, 640]
    w = gen.workload_varlen_prefill(lens=lens, hq=2, hk=1, head_dim=64, page_size=128)
    # rebuild the cache inside a pool of 2,100 pages (268,800 slots); the sequences' pages are scattered through it
    pool = 2100
    perm = torch.randperm(pool, generator=g)[:w["k_cache"].shape[0]]
    kc = torch.full((pool, 128, 1, 64), float("nan"), dtype=torch.bfloat16)
    vc = torch.full((pool, 128, 1, 64), float("nan"), dtype=torch.bfloat16)
    kc[perm], vc[perm] = w["k_cache"], w["v_cache"]
    idx = perm[w["kv_page_indices"].long()].to(torch.int32)
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(kc), dev(vc), dev(w["cu_seqlens_q"]), dev(w["kv_indptr"]), dev(idx),
                                dev(w["kv_last_page_lens"]), max_seqlen_q=w["max_seqlen_q"], scale=w["scale"])
    assert _lib.load().fck_fmha_last_kernel() == b"prefill_pp_kernel<uniform_page>"
    ro = orc.fmha_fwd(w["q"], kc, vc, seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"], kv_page_indices=idx,
                      kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "large pool")


def test_prefill_sequence_longer_than_the_page_cache(fmha, orc):
    """More key tiles than the kernel's per-workgroup page cache holds (4096 tiles = 262,144 keys): the tiles past the
    cache are looked up one by one.  300 queries at the end of a 263,000-key sequence (chunked prefill), one KV head."""
    g = torch.Generator().manual_seed(41)
    L, sq = 263000, 300
    kv = gen.paged_kv([L], 1, 64, torch.bfloat16, g, 128)
    q = gen.randn((1, sq, 2, 64), torch.bfloat16, g)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]))
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=2,
                      window=(-1, 0))
    assert_close(o, ro, 2e-2, "very long sequence")


@pytest.mark.parametrize("d", [64, 128])
def test_prefill_midsize_every_row(fmha, orc, d):
    """Every row of a 5,000-token sequence against the oracle: 79 key tiles per row tile at the end, so the 64-tile
    chunks of the first-row cache are reloaded, the 4-deep K/V rings wrap many times and 20 row tiles of 256 rows
    (the last one ragged) are all compared.  A second, short sequence shares the launch."""
    w = gen.workload_varlen_prefill(seed=61 + d, lens=[5000, 300], hq=2, hk=1, head_dim=d)
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), dev(w["cu_seqlens_q"]), dev(w["kv_indptr"]),
                                dev(w["kv_page_indices"]), dev(w["kv_last_page_lens"]), max_seqlen_q=w["max_seqlen_q"],
                                scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "mid-size, every row")


def _sample_rows(L, g):
    """Rows of a length-L sequence worth checking: both ends, the borders of the 32-row wave, 128-row group and 256-row
    workgroup tiles, the middle, four random 256-row borders and 32 random rows."""
    rows = {0, 31, 32, 127, 128, 255, 256, 257, L // 2 - 1, L // 2, L // 2 + 1, L - 1}
    nt = max(L // 256, 1)
    for k in torch.randint(1, nt + 1, (4,), generator=g).tolist():
        rows.update({256 * k - 1, 256 * k, 256 * k + 1})
    rows.update(torch.randint(0, L, (32,), generator=g).tolist())
    return sorted(r for r in rows if 0 <= r < L)


@pytest.mark.parametrize("d", [128, 256])
def test_workload5_full(fmha, orc, d):
    """Full-size varlen causal prefill (config 5).  The oracle cannot run 3 TFLOP, so it checks a stratified sample of
    rows of every sequence (about 50 per sequence, see _sample_rows): row i of a causal sequence is a one-query problem
    over its first i + 1 keys, run through the same block table.  The decode kernel (an independent code path)
    re-computes the last row of each sequence as well."""
    w = gen.workload_varlen_prefill(head_dim=d)
    args = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fmha.fmha_batch_prefill(*args, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"]).cpu()
    assert torch.isfinite(o.float()).all()
    cu, lens, B = w["cu_seqlens_q"].tolist(), w["lens"], len(w["lens"])
    g = torch.Generator().manual_seed(500 + d)
    qs, got, tbl, sl = [], [], [], []
    for b in range(B):
        for i in _sample_rows(lens[b], g):
            qs.append(w["q"][cu[b] + i])
            got.append(o[cu[b] + i])
            tbl.append(w["block_table"][b])
            sl.append(i + 1)
    q1 = torch.stack(qs).unsqueeze(1).contiguous()  # [rows, 1, Hq, D]: each sampled row is its own one-query sequence
    ro = orc.fmha_fwd(q1, w["k_cache"], w["v_cache"], seqlen_k=torch.tensor(sl, dtype=torch.int32),
                      block_table=torch.stack(tbl).contiguous(), scale=w["scale"])
    assert_close(torch.stack(got).unsqueeze(1), ro, 2e-2, f"{len(qs)} sampled rows")
    # cross-kernel: the decode path on the last query of each sequence
    qlast = torch.stack([w["q"][cu[b + 1] - 1] for b in range(B)]).unsqueeze(1).contiguous()
    od = fmha.fmha_decode_paged(dev(qlast), args[1], args[2], dev(w["seqlen_k"]), dev(w["block_table"]), num_splits=4,
                                scale=w["scale"]).cpu()
    last = torch.stack([o[cu[b + 1] - 1] for b in range(B)]).unsqueeze(1)
    assert_close(last, od, 2e-2, "prefill vs decode kernel")
