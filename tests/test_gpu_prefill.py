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


@pytest.mark.parametrize("d", [128, 256])
def test_workload5_full(fmha, orc, d):
    """Full-size varlen causal prefill.  The oracle cannot run 3 TFLOP; it checks the last 4 and the first 8 query
    rows of every sequence, and the decode kernel (an independent code path) re-computes the last row of each."""
    w = gen.workload_varlen_prefill(head_dim=d)
    args = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fmha.fmha_batch_prefill(*args, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"]).cpu()
    assert torch.isfinite(o.float()).all()
    cu, lens, B = w["cu_seqlens_q"].tolist(), w["lens"], len(w["lens"])
    # last 4 rows: a 4-query problem over all L keys (bottom-right causal)
    tail = torch.cat([w["q"][cu[b + 1] - 4:cu[b + 1]] for b in range(B)]).contiguous()
    cu4 = torch.arange(0, 4 * B + 1, 4, dtype=torch.int32)
    ro = orc.fmha_fwd(tail, w["k_cache"], w["v_cache"], seqstart_q=cu4, seqlen_k=w["seqlen_k"], block_table=w["block_table"],
                      scale=w["scale"], mask_type=2, window=(-1, 0))
    got = torch.cat([o[cu[b + 1] - 4:cu[b + 1]] for b in range(B)])
    assert_close(got, ro, 2e-2, "last rows")
    # first 8 rows: an 8x8 causal problem
    head = torch.cat([w["q"][cu[b]:cu[b] + 8] for b in range(B)]).contiguous()
    cu8 = torch.arange(0, 8 * B + 1, 8, dtype=torch.int32)
    ro = orc.fmha_fwd(head, w["k_cache"], w["v_cache"], seqstart_q=cu8, seqlen_k=torch.full((B,), 8, dtype=torch.int32),
                      block_table=w["block_table"], scale=w["scale"], mask_type=2, window=(-1, 0))
    got = torch.cat([o[cu[b]:cu[b] + 8] for b in range(B)])
    assert_close(got, ro, 2e-2, "first rows")
    # cross-kernel: the decode path on the last query of each sequence
    qlast = torch.stack([w["q"][cu[b + 1] - 1] for b in range(B)]).unsqueeze(1).contiguous()
    od = fmha.fmha_decode_paged(dev(qlast), args[1], args[2], dev(w["seqlen_k"]), dev(w["block_table"]), num_splits=4,
                                scale=w["scale"]).cpu()
    got = torch.stack([o[cu[b + 1] - 1] for b in range(B)]).unsqueeze(1)
    assert_close(got, od, 2e-2, "prefill vs decode kernel")
