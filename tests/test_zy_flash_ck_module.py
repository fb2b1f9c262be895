"""GPU: the compiled `flash_ck` module (torch tensors in and out, as the reference's pybind layer) against the oracle:
the dense fp16 benchmark workload (batch 2, 128 tokens, 8 heads, head dim 64) by module name, then one small case per operator."""
import math

import pytest
import torch

from flashck_amd import generators as gen
from helpers import ATOL, assert_bits_equal, assert_close, assert_lse_close, dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fck(fmha):
    import flash_ck  # raises with the build command when the compiled module is missing: no fallback
    return flash_ck


def test_config1_dense_fp16_by_module_name(fck, orc):
    w = gen.workload_dense_fp16()
    o = fck.fmha_fwd(dev(w["q"]), dev(w["k"]), dev(w["v"]), scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k"], w["v"], scale=w["scale"])
    assert o.dtype == torch.float16 and tuple(o.shape) == (2, 128, 8, 64)
    assert_close(o, ro, ATOL[torch.float16], "flash_ck.fmha_fwd")
    o2 = fck.ops.fmha.fmha_fwd(dev(w["q"]), dev(w["k"]), dev(w["v"]), scale=w["scale"])
    assert_bits_equal(o, o2, "compiled module vs functional API")


def test_varlen_causal(fck, orc):
    g = torch.Generator().manual_seed(4)
    lens = [5, 130, 64]
    cu = torch.tensor([0, 5, 135, 199], dtype=torch.int32)
    q, k, v = (gen.randn((sum(lens), h, 64), torch.bfloat16, g) for h in (4, 2, 2))
    o = fck.fmha_fwd_varlen(dev(q), dev(k), dev(v), dev(cu), dev(cu), 130, mask_type=2, window_left=-1, window_right=0)
    ro = orc.fmha_fwd(q, k, v, seqstart_q=cu, seqstart_k=cu, scale=0.125, mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "fmha_fwd_varlen")


def test_splitkv_combine_paged(fck, orc):
    w = gen.workload_paged_decode(seed=12, batch=3, hq=16, hk=4, head_dim=128, min_len=1, max_len=900)
    ns = fck.fmha_num_splits_heuristic(3, 16, 4, 1, 900, 128, 0)
    o_acc, lse_acc = fck.fmha_fwd_splitkv(dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"]), ns, dev(w["seqlen_k"]), dev(w["block_table"]),
                                          scale=w["scale"])
    o = fck.fmha_fwd_splitkv_combine(lse_acc, o_acc, torch.bfloat16)
    kw = dict(seqlen_k=w["seqlen_k"], block_table=w["block_table"], scale=w["scale"])
    ro_acc, rlse = orc.fmha_splitkv(w["q"], w["k_cache"], w["v_cache"], ns, **kw)
    assert_lse_close(lse_acc, rlse, what="lse_acc")
    assert_close(o_acc, ro_acc, 2e-2, "o_acc")
    assert_close(o, orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], **kw), 2e-2, "o")


def test_appendkv_bit_exact(fck, orc):
    w = gen.workload_appendkv_decode(batch=3, hq=8, hk=2, head_dim=128, min_len=10, max_len=300, max_new=5)
    q, kc, vc = dev(w["q"]), dev(w["k_cache"]), dev(w["v_cache"])
    fck.fmha_fwd_appendkv(q, kc, vc, dev(w["knew"]), dev(w["vnew"]), dev(w["seqlen_k"]), dev(w["block_table"]),
                          cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=w["max_new"], rotary_cos=dev(w["rotary_cos"]),
                          rotary_sin=dev(w["rotary_sin"]), rope_mode=2, has_mask=True)
    q_ref, kc_ref, vc_ref = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    orc.appendkv(q_ref, kc_ref, vc_ref, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], w["rotary_cos"], w["rotary_sin"],
                 rope_mode=orc.ROPE_HALF_ROTATED, has_mask=True, block_table=w["block_table"])
    assert_bits_equal(kc, kc_ref, "k_cache")
    assert_bits_equal(vc, vc_ref, "v_cache")
    assert_bits_equal(q, q_ref, "q")


def test_batch_prefill_and_pagedkv(fck, orc):
    w = gen.workload_varlen_prefill(seed=5, batch=3, hq=8, hk=2, head_dim=128, min_len=20, max_len=400)
    a = [dev(w[k]) for k in ("q", "k_cache", "v_cache", "cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fck.fmha_batch_prefill(*a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"])
    ro = orc.fmha_fwd(w["q"], w["k_cache"], w["v_cache"], seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"],
                      kv_page_indices=w["kv_page_indices"], kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=2, window=(-1, 0))
    assert_close(o, ro, 2e-2, "fmha_batch_prefill")
    # the same sequences through a block table
    lens = w["lens"]
    width = max(int(w["kv_indptr"][i + 1] - w["kv_indptr"][i]) for i in range(len(lens)))
    bt = torch.zeros(len(lens), width, dtype=torch.int32)
    for i in range(len(lens)):
        p = w["kv_page_indices"][w["kv_indptr"][i]:w["kv_indptr"][i + 1]]
        bt[i, :p.numel()] = p
    sl = torch.tensor(lens, dtype=torch.int32)
    o2 = fck.fmha_fwd_pagedkv(a[0], a[1], a[2], dev(sl), dev(bt), cu_seqlens_q=a[3], max_seqlen_q=w["max_seqlen_q"], scale=w["scale"])
    assert_close(o2, ro, 2e-2, "fmha_fwd_pagedkv")


def test_e4m3_tensors_take_the_all_fp8_roles(fck):
    """float8_e4m3fn q / k / v through the compiled module: the two-key closed form (88 with the cast of P, 96 without;
    see test_zx_fp8_roles) on the dense call and on split-KV + combine."""
    f8 = torch.float8_e4m3fn
    q = torch.zeros(1, 1, 1, 64)
    q[..., 0] = 1.0
    k = torch.zeros(1, 2, 1, 64)
    k[0, 1, 0, 0] = -1.25
    v = torch.zeros(1, 2, 1, 64)
    v[0, 1] = 416.0
    q, k, v = dev(q.to(f8)), dev(k.to(f8)), dev(v.to(f8))
    o = fck.fmha_fwd(q, k, v, scale=1.0)
    assert o.dtype == f8 and torch.all(o.cpu().float() == 88.0), o.cpu().float().unique()
    # the same two keys as the first rows of a one-page cache
    kc, vc = torch.zeros(1, 64, 1, 64), torch.zeros(1, 64, 1, 64)
    kc[0, :2], vc[0, :2] = k[0].float().cpu(), v[0].float().cpu()
    o_acc, lse_acc = fck.fmha_fwd_splitkv(q, dev(kc.to(f8)), dev(vc.to(f8)), 1, dev(torch.tensor([2], dtype=torch.int32)),
                                          dev(torch.zeros(1, 1, dtype=torch.int32)), scale=1.0)
    o = fck.fmha_fwd_splitkv_combine(lse_acc, o_acc, f8)
    assert o.dtype == f8 and torch.all(o.cpu().float() == 88.0), o.cpu().float().unique()
