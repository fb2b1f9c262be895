"""GPU: the debug checker of paged-cache arguments (fck_fmha_validate_paged) and the ticket reset of the fused entry."""
import pytest
import torch

from flashck_amd import generators as gen
from flashck_amd.utils import flags
from helpers import assert_close, dev

pytestmark = pytest.mark.gpu


def _kv(lens, page=16, hk=2, d=64, seed=3):
    g = torch.Generator().manual_seed(seed)
    return gen.paged_kv(lens, hk, d, torch.bfloat16, g, page)


def test_block_table_checks(fmha):
    kv = _kv([1, 16, 17, 100, 33])
    bt, sl, pool = kv["block_table"], kv["seqlen_k"], kv["k_cache"].shape[0]
    run = lambda s, t: fmha.validate_paged(seqlen_k=dev(s), block_table=dev(t), num_total_pages=pool, page_size=16).cpu().tolist()
    assert run(sl, bt) == [0, 0, 0, -1]
    too_long = sl.clone()
    too_long[3] = bt.shape[1] * 16 + 1            # one key more than the table row can address
    assert run(too_long, bt) == [1, 0, 0, 3]
    negative = sl.clone()
    negative[1] = -5
    assert run(negative, bt) == [1, 0, 0, 1]
    bad = bt.clone()
    bad[2, 1] = pool                                # first id past the pool, in an entry sequence 2 uses (17 keys = 2 pages)
    bad[4, 0] = -1
    assert run(sl, bad) == [0, 2, 0, 2]
    unused = bt.clone()
    unused[0, 1:] = 10 ** 6                         # entries behind a sequence's last page are never read
    assert run(sl, unused) == [0, 0, 0, -1]
    # full capacity is fine
    full = sl.clone()
    full[3] = bt.shape[1] * 16
    assert run(full, bt)[0] == 0


def test_page_list_checks(fmha):
    indptr = torch.tensor([0, 2, 2, 5], dtype=torch.int32)
    pages = torch.tensor([4, 0, 7, 1, 3], dtype=torch.int32)
    last = torch.tensor([16, 16, 5], dtype=torch.int32)
    run = lambda i, p, l: fmha.validate_paged(kv_indptr=dev(i), kv_page_indices=dev(p), kv_last_page_lens=dev(l) if l is not None else None,
                                              num_total_pages=8, page_size=16).cpu().tolist()
    assert run(indptr, pages, last) == [0, 0, 0, -1]
    assert run(indptr, pages, None) == [0, 0, 0, -1]
    assert run(indptr, torch.tensor([4, 0, 8, 1, 3], dtype=torch.int32), last) == [0, 1, 0, 2]
    assert run(indptr, pages, torch.tensor([16, 16, 17], dtype=torch.int32)) == [0, 0, 1, 2]
    assert run(indptr, pages, torch.tensor([0, 16, 5], dtype=torch.int32)) == [0, 0, 1, 0]
    assert run(torch.tensor([0, 3, 2, 5], dtype=torch.int32), pages, last) == [0, 0, 1, 1]   # not monotone


def test_debug_flag_makes_the_operators_check(fmha, orc):
    kv = _kv([40, 9], page=16, hk=2, d=64)
    g = torch.Generator().manual_seed(1)
    q = gen.randn((2, 1, 4, 64), torch.bfloat16, g)
    args = (dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]))
    bad_len = kv["seqlen_k"].clone()
    bad_len[1] = kv["block_table"].shape[1] * 16 + 3
    flags.set_flag_value("FC_DEBUG_KERNEL_INSTANCE", "true")
    try:
        with pytest.raises(ValueError, match="first offending sequence: 1"):
            fmha.fmha_fwd_splitkv(*args, 2, seqlen_k=dev(bad_len), block_table=dev(kv["block_table"]))
        with pytest.raises(ValueError, match="page id"):
            bad = kv["block_table"].clone()
            bad[0, 0] = 10 ** 5
            fmha.fmha_fwd_pagedkv(*args, dev(kv["seqlen_k"]), dev(bad))
        # consistent arguments pass through the check and give the usual result
        o = fmha.fmha_decode_paged(*args, dev(kv["seqlen_k"]), dev(kv["block_table"]), num_splits=2)
    finally:
        flags.set_flag_value("FC_DEBUG_KERNEL_INSTANCE", "false")
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=0.125)
    assert_close(o, ro, 2e-2, "decode under the debug flag")


def test_fused_reset_leaves_the_fused_path_working(fmha, orc):
    kv = _kv([300, 77, 1], page=16, hk=2, d=64, seed=8)
    g = torch.Generator().manual_seed(2)
    q = gen.randn((3, 1, 8, 64), torch.bfloat16, g)
    args = (dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]))
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=0.125)
    for _ in range(2):
        fmha.fused_reset()
        o = fmha.fmha_fwd_splitkv_fused(*args, 3, seqlen_k=dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]))
        assert_close(o, ro, 2e-2, "fused after reset")
