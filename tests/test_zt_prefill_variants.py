"""GPU: the tile variants of the ping-pong prefill kernel (fck_fmha_attrs.prefill_variant) and their tuner."""
import pytest
import torch

from flashck_amd import _lib, generators as gen
from flashck_amd.utils import flags, tuning
from helpers import ATOL, assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu

NAMES = {1: b"prefill_pp_kernel<uniform_page>", 2: b"prefill_pp_kernel<uniform_page,fast_requests>",
         3: b"prefill_pp_kernel<uniform_page,max_in_matrix_phase>", 4: b"prefill_pp_kernel<uniform_page,fast_requests,max_in_matrix_phase>"}


def _workload(d, page, dtype, lens=(300, 700, 129, 1)):
    w = gen.workload_varlen_prefill(seed=70 + d + page, batch=len(lens), hq=4, hk=2, head_dim=d, page_size=page, dtype=dtype, lens=list(lens))
    a = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    return w, a


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,page", [(128, 128), (128, 64), (64, 64)])
@pytest.mark.parametrize("mask", [(2, (-1, 0)), (0, (-1, -1)), (2, (150, 0))])
def test_every_variant_matches_the_oracle_and_the_default(fmha, orc, dtype, d, page, mask):
    w, a = _workload(d, page, dtype)
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=mask[0],
                      window=mask[1])
    base = None
    for variant in (1, 2, 3, 4):
        o = fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], mask_type=mask[0], window=mask[1],
                                    prefill_variant=variant)
        assert _lib.load().fck_fmha_last_kernel() == NAMES[variant]
        assert_close(o, ro, ATOL[dtype], f"variant {variant}")
        if base is None:
            base = o.clone()
        else:
            assert_bits_equal(o, base, f"variant {variant} against the default schedule")   # same arithmetic, other schedule


def test_variant_through_the_block_table_entry_point(fmha, orc):
    g = torch.Generator().manual_seed(5)
    kv = gen.paged_kv([260, 400], 2, 128, torch.bfloat16, g, 128)
    q = gen.randn((2, 260, 8, 128), torch.bfloat16, g)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(kv["k_cache"]), dev(kv["v_cache"]), dev(kv["seqlen_k"]), dev(kv["block_table"]), prefill_variant=4)
    assert _lib.load().fck_fmha_last_kernel() == NAMES[4]
    ro = orc.fmha_fwd(q, kv["k_cache"], kv["v_cache"], seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "variant 4, block table")


def test_variants_the_problem_cannot_take_are_refused(fmha):
    w, a = _workload(256, 64, torch.bfloat16, lens=(200, 140))
    with pytest.raises(ValueError, match="needs the ping-pong kernel"):
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], prefill_variant=2)            # head dim 256
    w, a = _workload(128, 48, torch.bfloat16, lens=(200, 140))
    with pytest.raises(ValueError, match="needs the ping-pong kernel"):
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], prefill_variant=3)            # pages of 48 keys
    w, a = _workload(128, 128, torch.bfloat16, lens=(100, 90))
    with pytest.raises(ValueError, match="needs the ping-pong kernel"):
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], prefill_variant=4)            # short query runs
    with pytest.raises(ValueError):
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], prefill_variant=5)
    fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], prefill_variant=1)                # the default schedule fits every call


def test_tuner_records_a_variant_and_later_calls_use_it(fmha, tmp_path, monkeypatch):
    w, a = _workload(128, 128, torch.bfloat16)
    cache = tuning.TuningCache(str(tmp_path))
    monkeypatch.setattr(tuning, "default_cache", lambda: cache)
    flags.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "1")
    flags.set_flag_value("FC_TUNING_NUM_REPEATS", "2")
    try:
        rec = fmha.tune_prefill_variant(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], cache=cache)
        assert rec["variant"] in (1, 2, 3, 4) and set(rec["tried_us"]) == {"v1", "v2", "v3", "v4"} and rec["kernel"].encode() == NAMES[rec["variant"]]
        fmha.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"])             # prefill_variant = 0: the record
        assert _lib.load().fck_fmha_last_kernel() == NAMES[rec["variant"]]
        # the same class of problems with pages the variants cannot take falls back to the library's choice
        w2, a2 = _workload(128, 128, torch.bfloat16, lens=(100, 128, 64, 2))
        fmha.fmha_batch_prefill(*a2, max_seqlen_q=w2["max_seqlen_q"], scale=w2["scale"])
    finally:
        flags.set_flag_value("FC_TUNING_NUM_COLD_ITERATION", "16")
        flags.set_flag_value("FC_TUNING_NUM_REPEATS", "64")
