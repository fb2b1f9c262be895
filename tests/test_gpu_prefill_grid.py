"""GPU parity of the direct-to-LDS prefill kernels against the CPU oracle on workloads with many workgroups per CU:
several row tiles and heads per sequence, mixed lengths, every mask kind, repeated launches; head dims 64 / 128
(ping-pong kernel) and 256 (4-wave direct-to-LDS kernel)."""
import pytest
import torch

from flashck_amd import generators as gen
from helpers import ATOL, assert_close, dev

pytestmark = pytest.mark.gpu


def _check(fmha, orc, w, dtype, what):
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), dev(w["cu_seqlens_q"]), dev(w["kv_indptr"]),
                                dev(w["kv_page_indices"]), dev(w["kv_last_page_lens"]), max_seqlen_q=w["max_seqlen_q"],
                                scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"],
                      mask_type=2, window=(-1, 0))
    assert_close(o, ro, ATOL[dtype], what)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("page", [64, 128])
def test_few_items_per_workgroup(fmha, orc, dtype, d, page):
    # 5 sequences x 4 heads x at most 2 row tiles
    w = gen.workload_varlen_prefill(seed=150 + d + page, batch=5, hq=4, hk=2, head_dim=d, min_len=129, max_len=400,
                                    page_size=page, dtype=dtype)
    _check(fmha, orc, w, dtype, "few workgroups")


@pytest.mark.parametrize("d", [64, 128])
def test_many_items_per_workgroup(fmha, orc, d):
    # 48 sequences x 16 heads x up to 5 row tiles: several workgroups per CU (lengths from 130 rows = 3 key tiles up)
    w = gen.workload_varlen_prefill(seed=160 + d, batch=48, hq=16, hk=4, head_dim=d, min_len=130, max_len=1200,
                                    page_size=64, dtype=torch.bfloat16)
    _check(fmha, orc, w, torch.bfloat16, "many workgroups")


def test_short_and_long_sequences_mixed(fmha, orc):
    # one-tile and two-tile sequences between long ones, max_seqlen_q far above most lengths
    g = torch.Generator().manual_seed(170)
    lens = [1, 2000, 63, 64, 65, 1500, 129, 257, 700, 130, 5, 1999]
    w = gen.workload_varlen_prefill(seed=170, batch=len(lens), hq=8, hk=8, head_dim=128, min_len=1, max_len=2000,
                                    page_size=128, dtype=torch.bfloat16, lens=lens)
    _check(fmha, orc, w, torch.bfloat16, "mixed lengths")


@pytest.mark.parametrize("mask", [(0, (-1, -1)), (2, (-1, 0)), (2, (100, 0)), (1, (-1, 0))])
def test_dense_batch_mode_masks(fmha, orc, mask):
    # no page table: contiguous K/V, every mask kind, sliding window (row tiles that start past tile 0)
    g = torch.Generator().manual_seed(180)
    q = gen.randn((3, 700, 8, 128), torch.bfloat16, g)
    k = gen.randn((3, 900, 2, 128), torch.bfloat16, g)
    v = gen.randn((3, 900, 2, 128), torch.bfloat16, g)
    mt, win = mask
    o = fmha.fmha_fwd(dev(q), dev(k), dev(v), mask_type=mt, window=win)
    ro = orc.fmha_fwd(q, k, v, mask_type=mt, window=win)
    assert_close(o, ro, 2e-2, "dense, masks")


def test_repeated_launches_agree(fmha, orc):
    # the kernel keeps no state between launches: the same call twice gives the same bits
    w = gen.workload_varlen_prefill(seed=190, batch=20, hq=8, hk=2, head_dim=128, min_len=200, max_len=900, page_size=128)
    args = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o1 = fmha.fmha_batch_prefill(*args, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"]).clone()
    o2 = fmha.fmha_batch_prefill(*args, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"])
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))



# ---- head dim 256 ----
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("page", [64, 128])
def test_dma256_paged(fmha, orc, dtype, page):
    w = gen.workload_varlen_prefill(seed=250 + page, batch=6, hq=4, hk=2, head_dim=256, min_len=1, max_len=700,
                                    page_size=page, dtype=dtype)
    _check(fmha, orc, w, dtype, "head dim 256, direct to LDS")


@pytest.mark.parametrize("mask", [(0, (-1, -1)), (2, (-1, 0)), (2, (90, 0)), (1, (-1, 0))])
def test_dma256_dense_masks(fmha, orc, mask):
    g = torch.Generator().manual_seed(260)
    q = gen.randn((2, 300, 4, 256), torch.bfloat16, g)
    k = gen.randn((2, 450, 2, 256), torch.bfloat16, g)
    v = gen.randn((2, 450, 2, 256), torch.bfloat16, g)
    mt, win = mask
    o = fmha.fmha_fwd(dev(q), dev(k), dev(v), mask_type=mt, window=win)
    ro = orc.fmha_fwd(q, k, v, mask_type=mt, window=win)
    assert_close(o, ro, 2e-2, "dense, head dim 256")
