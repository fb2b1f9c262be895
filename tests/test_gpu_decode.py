"""GPU parity: split-KV forward + LSE combine against the CPU oracle (called through the C ABI)."""
import math

import pytest
import torch

from flashck_amd import generators as gen
from helpers import ATOL, assert_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu


def _run_paged(fmha, orc, w, num_splits, mask_type=0, window=(-1, -1)):
    q, kc, vc = dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"])
    bt, sl = dev(w["block_table"]), dev(w["seqlen_k"])
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(q, kc, vc, num_splits, seqlen_k=sl, block_table=bt, scale=w["scale"],
                                           mask_type=mask_type, window=window)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype)
    torch.cuda.synchronize()
    kw = dict(seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"], mask_type=mask_type, window=window)
    ro_acc, rlse_acc = orc.fmha_splitkv(w["q"], w["k_cache"], w["v_cache"], num_splits, **kw)
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], **kw)
    atol = ATOL[q.dtype]
    assert_lse_close(lse_acc, rlse_acc, what="lse_acc")
    assert_close(o_acc, ro_acc, atol, "o_acc")
    assert_close(o, ro, atol, "o")
    return o


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hq,hk,d", [(8, 8, 64), (32, 8, 128), (64, 8, 128), (16, 2, 256), (4, 4, 128)])
@pytest.mark.parametrize("page,num_splits", [(128, 1), (128, 3), (16, 4), (64, 8)])
def test_paged_decode_small(fmha, orc, dtype, hq, hk, d, page, num_splits):
    w = gen.workload_paged_decode(seed=7 + hq + d + page, batch=3, hq=hq, hk=hk, head_dim=d, min_len=1, max_len=700,
                                  page_size=page, dtype=dtype)
    _run_paged(fmha, orc, w, num_splits)


@pytest.mark.parametrize("page", [128, 48])
def test_paged_decode_edge_lengths(fmha, orc, page):
    # lengths around tile and page borders, more splits than keys, a one-key sequence
    g = torch.Generator().manual_seed(3)
    lens = [1, 31, 32, 33, 127, 128, 129, 257]
    kv = gen.paged_kv(lens, 2, 128, torch.bfloat16, g, page)
    kv["q"] = gen.randn((len(lens), 1, 8, 128), torch.bfloat16, g)
    kv["scale"] = 1 / math.sqrt(128)
    for ns in (1, 2, 8):
        _run_paged(fmha, orc, kv, ns)


@pytest.mark.parametrize("sq,hq,hk", [(4, 8, 2), (16, 32, 8), (3, 4, 4), (7, 16, 2)])
def test_paged_multi_query_causal(fmha, orc, sq, hq, hk):
    # several query rows per sequence, bottom-right causal: the decode that follows an append of sq tokens
    g = torch.Generator().manual_seed(11 + sq)
    lens = [sq, sq + 5, 300, 129]
    kv = gen.paged_kv(lens, hk, 128, torch.bfloat16, g, 128)
    kv["q"] = gen.randn((len(lens), sq, hq, 128), torch.bfloat16, g)
    kv["scale"] = 1 / math.sqrt(128)
    for ns in (1, 3):
        _run_paged(fmha, orc, kv, ns, mask_type=2, window=(-1, 0))
    _run_paged(fmha, orc, kv, 2, mask_type=1, window=(-1, 0))      # top-left causal
    _run_paged(fmha, orc, kv, 2, mask_type=2, window=(17, 0))      # sliding window


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,page", [(128, 128), (64, 64), (128, 48)])
def test_paged_decode_head_pairs(fmha, orc, dtype, d, page):
    """Grids of at least one workgroup per CU take the kernel that streams two KV heads per workgroup (16-key tiles):
    20 sequences x 8 KV heads x 4 splits.  Lengths around the 16-key tile and page borders; page 48 is not a multiple
    of the tile, so it takes the per-row lookup variant."""
    g = torch.Generator().manual_seed(31 + d + page)
    lens = [1, 15, 16, 17, 47, 48, 49, 95, 96, 97, 127, 128, 129, 255, 256, 257, 700, 1023, 1500, 33]
    kv = gen.paged_kv(lens, 8, d, dtype, g, page)
    kv["q"] = gen.randn((len(lens), 1, 32, d), dtype, g)
    kv["scale"] = 1 / math.sqrt(d)
    _run_paged(fmha, orc, kv, 4)
    from flashck_amd import _lib
    assert b"head_pairs" in _lib.load().fck_fmha_last_kernel()   # the name says which variant the launcher took
    _run_paged(fmha, orc, kv, 4, mask_type=2, window=(40, 0))  # sliding window: leading tiles are skipped


def test_decode_paged_fused_flag(fmha, orc):
    """fmha_decode_paged(fused=True) = one launch; same result as the two-launch path within the output tolerance."""
    w = gen.workload_paged_decode(seed=91, batch=5, hq=32, hk=8, head_dim=128, min_len=1, max_len=3000)
    args = (dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), dev(w["seqlen_k"]), dev(w["block_table"]))
    o1 = fmha.fmha_decode_paged(*args, num_splits=0, max_seqlen_k=3000, scale=w["scale"], fused=True)
    o2 = fmha.fmha_decode_paged(*args, num_splits=0, max_seqlen_k=3000, scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"])
    assert_close(o1, ro, 2e-2, "fused")
    assert_close(o2, ro, 2e-2, "two launches")


def test_group_mode_ragged_queries(fmha, orc):
    # ragged query counts (1..16 new tokens per sequence) through seqstart_q
    g = torch.Generator().manual_seed(5)
    qn = [1, 16, 5, 9]
    lens = [200, 77, 1030, 16]
    hq, hk, d = 32, 8, 128
    kv = gen.paged_kv(lens, hk, d, torch.bfloat16, g, 128)
    cu = torch.zeros(len(qn) + 1, dtype=torch.int32)
    cu[1:] = torch.tensor(qn).cumsum(0)
    q = gen.randn((sum(qn), hq, d), torch.bfloat16, g)
    scale = 1 / math.sqrt(d)
    for ns in (1, 4):
        o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), ns, seqlen_k=dev(kv["seqlen_k"]),
                                               block_table=dev(kv["block_table"]), cu_seqlens_q=dev(cu), max_seqlen_q=16,
                                               scale=scale, mask_type=2, window=(-1, 0))
        o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype, cu_seqlens_q=dev(cu), max_seqlen_q=16)
        kw = dict(seqstart_q=cu, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale, mask_type=2, window=(-1, 0))
        ro_acc, rlse = orc.fmha_splitkv(q, kv["k_cache"], kv["v_cache"], ns, **kw)
        ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], **kw)
        assert_lse_close(lse_acc, rlse, what="lse_acc")
        assert_close(o_acc, ro_acc, 2e-2, "o_acc")
        assert_close(o, ro, 2e-2, "o")


def test_batch_cache_with_cache_batch_idx(fmha, orc):
    # non-paged cache [rows, sk, Hk, D] addressed through cache_batch_idx
    g = torch.Generator().manual_seed(9)
    B, sk, hq, hk, d = 3, 200, 8, 2, 128
    k = gen.randn((5, sk, hk, d), torch.float16, g)
    v = gen.randn((5, sk, hk, d), torch.float16, g)
    q = gen.randn((B, 1, hq, d), torch.float16, g)
    idx = torch.tensor([4, 0, 2], dtype=torch.int32)
    sl = torch.tensor([200, 1, 150], dtype=torch.int32)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(q), dev(k), dev(v), 4, seqlen_k=dev(sl), cache_batch_idx=dev(idx))
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, q.dtype)
    ro = orc.fmha_fwd(q, k, v, seqlen_k=sl, cache_batch_idx=idx, batch=B)
    assert_close(o, ro, 1e-2, "o")


@pytest.mark.parametrize("variant,num_splits,batch", [(1, 1, 48), (1, 2, 30), (2, 3, 30), (1, 1, 64)])
def test_ragged_batch_taken_longest_first(fmha, orc, variant, num_splits, batch):
    # between one and two workgroups per CU the kernel deals its workgroup ids to the sequences in order of decreasing
    # length (equal lengths: in index order); every sequence must still come out in its own place
    g = torch.Generator().manual_seed(41 + batch)
    lens = gen.randint_list(1, 300, batch, g)
    lens[3] = lens[7] = lens[11] = max(lens)  # ties, also for the first place
    lens[5] = lens[6] = 1
    kv = gen.paged_kv(lens, 8, 128, torch.bfloat16, g, 64)
    kv["q"] = gen.randn((batch, 1, 32, 128), torch.bfloat16, g)
    scale = 1 / math.sqrt(128)
    args = dict(seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]), scale=scale)
    o_acc, lse_acc = fmha.fmha_fwd_splitkv(dev(kv["q"]), dev(kv["k_cache"]), dev(kv["v_cache"]), num_splits, decode_variant=variant, **args)
    o = fmha.fmha_fwd_splitkv_combine(lse_acc, o_acc, torch.bfloat16)
    torch.cuda.synchronize()
    kw = dict(seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale)
    ro_acc, rlse_acc = orc.fmha_splitkv(kv["q"], kv["k_cache"], kv["v_cache"], num_splits, **kw)
    assert_lse_close(lse_acc, rlse_acc, what="lse_acc")
    assert_close(o_acc, ro_acc, ATOL[torch.bfloat16], "o_acc")
    assert_close(o, orc.fmha_fwd(kv["q"], kv["k_cache"], kv["v_cache"], **kw), ATOL[torch.bfloat16], "o")


def test_workload2_full(fmha, orc):
    w = gen.workload_paged_decode()
    ns = fmha.num_splits_heuristic(32, 32, 8, 1, max(w["lens"]), 128)
    o = _run_paged(fmha, orc, w, ns)
    # property: the result does not depend on the split count
    o1 = _run_paged(fmha, orc, w, 1)
    assert_close(o, o1, 2e-2, "split invariance")


def test_workload3_full(fmha, orc):
    w = gen.workload_splitkv_decode()
    _run_paged(fmha, orc, w, w["num_splits"])
