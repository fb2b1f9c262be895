"""GPU: the quantised (fp8 e4m3, static scales) K/V cache end to end: appendKV writes it bit-exactly as the oracle
does, the prefill entry points and the split-KV path read it, and a decode step chains the two."""
import math

import pytest
import torch

import helpers
from flashck_amd import _lib, generators as gen
from helpers import ATOL, assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu


def _bytes_equal(a, b, what):
    a, b = a.view(torch.uint8).cpu(), b.view(torch.uint8).cpu()
    bad = (a != b).nonzero()
    assert bad.numel() == 0, f"{what}: {bad.shape[0]} of {a.numel()} bytes differ, first at {bad[0].tolist()}"


def _fp8_pool(shape, fill=0x55):
    return torch.full(shape, fill, dtype=torch.uint8).view(torch.float8_e4m3fn)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rope_mode", [0, 1, 2])
@pytest.mark.parametrize("page", [16, 128])
def test_appendkv_fp8_cache_bit_exact(fmha, orc, dtype, rope_mode, page):
    """Whole pool compared byte for byte (appended rows quantised, everything else untouched), rotated q bit-exact."""
    w = gen.workload_appendkv_decode(seed=60 + page + rope_mode, batch=5, hq=8, hk=2, head_dim=128, min_len=1, max_len=700, max_new=9,
                                     page_size=page, dtype=dtype)
    kd, vd = 0.03, 0.021
    q, kc, vc = dev(w["q"]), dev(_fp8_pool(w["k_cache"].shape)), dev(_fp8_pool(w["v_cache"].shape))
    fmha.fmha_fwd_appendkv(q, kc, vc, dev(w["knew"]), dev(w["vnew"]), dev(w["seqlen_k"]), cu_seqlens_knew=dev(w["cu_seqlens_knew"]),
                           max_seqlen_knew=w["max_new"], rotary_cos=dev(w["rotary_cos"]), rotary_sin=dev(w["rotary_sin"]),
                           rope_mode=rope_mode, has_mask=True, block_table=dev(w["block_table"]), k_descale=kd, v_descale=vd)
    q_ref, kc_ref, vc_ref = w["q"].clone(), _fp8_pool(w["k_cache"].shape), _fp8_pool(w["v_cache"].shape)
    orc.appendkv(q_ref, kc_ref, vc_ref, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos=w["rotary_cos"], sin=w["rotary_sin"],
                 rope_mode=rope_mode, has_mask=True, block_table=w["block_table"], k_descale=kd, v_descale=vd)
    _bytes_equal(kc, kc_ref, "k_cache")
    _bytes_equal(vc, vc_ref, "v_cache")
    assert_bits_equal(q, q_ref, "q")


def test_appendkv_fp8_saturates_and_uniform_batch_form(fmha, orc):
    """[B, n, H, D] inputs without cu_seqlens; values far beyond 448 * descale land on +-448."""
    g = torch.Generator().manual_seed(3)
    B, n, hk, d = 2, 3, 2, 64
    kv = gen.paged_kv([20, 33], hk, d, torch.bfloat16, g, 16, capacity=[20 + n, 33 + n])
    knew = gen.randn((B, n, hk, d), torch.bfloat16, g) * 40
    vnew = gen.randn((B, n, hk, d), torch.bfloat16, g) * 40
    kc, vc = dev(_fp8_pool(kv["k_cache"].shape, 0)), dev(_fp8_pool(kv["v_cache"].shape, 0))
    fmha.fmha_fwd_appendkv(None, kc, vc, dev(knew), dev(vnew), dev(kv["seqlen_k"]), block_table=dev(kv["block_table"]),
                           k_descale=0.05, v_descale=0.05)
    kc_ref, vc_ref = _fp8_pool(kv["k_cache"].shape, 0), _fp8_pool(kv["v_cache"].shape, 0)
    cu = torch.tensor([0, n, 2 * n], dtype=torch.int32)
    orc.appendkv(None, kc_ref, vc_ref, knew.view(-1, hk, d), vnew.view(-1, hk, d), kv["seqlen_k"], cu, block_table=kv["block_table"],
                 k_descale=0.05, v_descale=0.05)
    _bytes_equal(kc, kc_ref, "k_cache")
    _bytes_equal(vc, vc_ref, "v_cache")
    assert (kc_ref.view(torch.uint8) & 0x7f == 0x7e).any(), "the case is meant to saturate"


def _quantised(w, kd, vd):
    return (w["k_cache"].float() / kd).to(torch.float8_e4m3fn), (w["v_cache"].float() / vd).to(torch.float8_e4m3fn)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d,page", [(128, 128), (64, 64), (256, 64), (128, 16)])
def test_batch_prefill_reads_fp8_cache(fmha, orc, dtype, d, page):
    w = gen.workload_varlen_prefill(seed=31 + d + page, batch=3, hq=8, hk=2, head_dim=d, min_len=1, max_len=330, page_size=page, dtype=dtype)
    kd, vd = 0.03, 0.025
    k8, v8 = _quantised(w, kd, vd)
    a = [dev(w[k]) for k in ("cu_seqlens_q", "kv_indptr", "kv_page_indices", "kv_last_page_lens")]
    o = fmha.fmha_batch_prefill(dev(w["q"]), dev(k8), dev(v8), *a, max_seqlen_q=w["max_seqlen_q"], scale=w["scale"], k_descale=kd, v_descale=vd)
    assert b"kv_fp8" in _lib.load().fck_fmha_last_kernel()
    ro = orc.fmha_fwd(w["q"], k8, v8, seqstart_q=w["cu_seqlens_q"], kv_indptr=w["kv_indptr"], kv_page_indices=w["kv_page_indices"],
                      kv_last_page_lens=w["kv_last_page_lens"], scale=w["scale"], mask_type=2, window=(-1, 0), k_descale=kd, v_descale=vd)
    assert_close(o, ro, ATOL[dtype], "batch prefill over an fp8 cache")


def test_pagedkv_prefill_reads_fp8_cache_with_alibi_and_window(fmha, orc):
    g = torch.Generator().manual_seed(17)
    dtype, hq, hk, d, sq = torch.bfloat16, 8, 4, 128, 70
    lens = [70, 200, 131]
    kv = gen.paged_kv(lens, hk, d, dtype, g, 64)
    kd, vd = 0.04, 0.03
    k8, v8 = _quantised(kv, kd, vd)
    q = gen.randn((3, sq, hq, d), dtype, g)
    slopes = (torch.rand(hq, generator=g) * 0.1).float()
    scale = 1 / math.sqrt(d)
    o = fmha.fmha_fwd_pagedkv(dev(q), dev(k8), dev(v8), dev(kv["seqlen_k"]), dev(kv["block_table"]), scale=scale, mask_type=2, window=(50, 0),
                              alibi_slopes=dev(slopes), k_descale=kd, v_descale=vd)
    ro = orc.fmha_fwd(q, k8, v8, seqlen_k=kv["seqlen_k"], block_table=kv["block_table"], scale=scale, mask_type=2, window=(50, 0),
                      alibi_slopes=slopes, k_descale=kd, v_descale=vd)
    assert_close(o, ro, ATOL[dtype], "paged prefill over an fp8 cache with ALiBi")


def test_decode_step_over_fp8_cache(fmha, orc):
    """append (quantising) -> split-KV over the quantised cache -> combine, as one step; against the oracle's chain."""
    w = gen.workload_appendkv_decode(seed=9, batch=4, hq=16, hk=4, head_dim=128, min_len=30, max_len=900, max_new=4, page_size=128)
    kd, vd = 0.03, 0.03
    k8, v8 = _quantised(w, kd, vd)
    q, kc, vc = dev(w["q"]), dev(k8), dev(v8)
    o, seqlen_new = fmha.fmha_decode_step(q, dev(w["knew"]), dev(w["vnew"]), kc, vc, dev(w["seqlen_k"]), dev(w["block_table"]),
                                          cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=w["max_new"],
                                          rotary_cos=dev(w["rotary_cos"]), rotary_sin=dev(w["rotary_sin"]), rope_mode=2, num_splits=3,
                                          scale=w["scale"], k_descale=kd, v_descale=vd)
    q_ref, k_ref, v_ref = w["q"].clone(), k8.clone(), v8.clone()
    orc.appendkv(q_ref, k_ref, v_ref, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos=w["rotary_cos"], sin=w["rotary_sin"],
                 rope_mode=2, has_mask=True, block_table=w["block_table"], k_descale=kd, v_descale=vd)
    sl_new = w["seqlen_k"] + torch.tensor(w["new"], dtype=torch.int32)
    ro = orc.fmha_fwd(q_ref, k_ref, v_ref, seqstart_q=w["cu_seqlens_knew"], seqlen_k=sl_new, block_table=w["block_table"], scale=w["scale"],
                      mask_type=2, window=(-1, 0), k_descale=kd, v_descale=vd)
    assert torch.equal(seqlen_new.cpu(), sl_new)
    _bytes_equal(kc, k_ref, "k_cache after the step")
    _bytes_equal(vc, v_ref, "v_cache after the step")
    assert_close(o, ro, 2e-2, "decode step over an fp8 cache")


def test_fp8_cache_argument_checks(fmha):
    w = gen.workload_appendkv_decode(seed=2, batch=1, hq=2, hk=1, head_dim=64, min_len=3, max_len=9, max_new=1, page_size=16)
    kc = dev(_fp8_pool(w["k_cache"].shape))
    args = (None, kc, kc.clone(), dev(w["knew"]), dev(w["vnew"]), dev(w["seqlen_k"]))
    kw = dict(cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=1, block_table=dev(w["block_table"]))
    with pytest.raises(ValueError, match="positive and finite"):
        fmha.fmha_fwd_appendkv(*args, k_descale=0.0, **kw)
    with pytest.raises(TypeError):   # one cache fp8, the other 16-bit
        fmha.fmha_fwd_appendkv(None, kc, dev(w["v_cache"]), *args[3:], **kw)


@pytest.mark.parametrize("with_idx", [True, False])
def test_appendkv_fp8_into_a_batch_cache(fmha, orc, with_idx):
    """A non-paged fp8 cache [slots, rows, Hk, D], addressed directly or through cache_batch_idx; packed, ragged new tokens."""
    g = torch.Generator().manual_seed(19)
    B, hk, hq, d, rows = 3, 2, 4, 64, 48
    new = [4, 1, 7]
    cu = torch.tensor([0, 4, 5, 12], dtype=torch.int32)
    knew, vnew = gen.randn((12, hk, d), torch.bfloat16, g), gen.randn((12, hk, d), torch.bfloat16, g)
    q = gen.randn((12, hq, d), torch.bfloat16, g)
    sl = torch.tensor([0, 36, 17], dtype=torch.int32)
    idx = torch.tensor([3, 1, 4], dtype=torch.int32) if with_idx else None
    cos, sin = gen.rotary_tables(rows + 1, d, torch.bfloat16)
    slots = 5 if with_idx else B
    q_ref, kc_ref, vc_ref = q.clone(), _fp8_pool((slots, rows, hk, d)), _fp8_pool((slots, rows, hk, d))
    orc.appendkv(q_ref, kc_ref, vc_ref, knew, vnew, sl, cu, cos, sin, rope_mode=2, has_mask=True, cache_batch_idx=idx, k_descale=0.04, v_descale=0.02)
    qd, kcd, vcd = dev(q.clone()), dev(_fp8_pool((slots, rows, hk, d))), dev(_fp8_pool((slots, rows, hk, d)))
    fmha.fmha_fwd_appendkv(qd, kcd, vcd, dev(knew), dev(vnew), dev(sl), cu_seqlens_knew=dev(cu), max_seqlen_knew=max(new), rotary_cos=dev(cos),
                           rotary_sin=dev(sin), rope_mode=2, cache_batch_idx=dev(idx), k_descale=0.04, v_descale=0.02)
    _bytes_equal(kcd, kc_ref, "k_cache")
    _bytes_equal(vcd, vc_ref, "v_cache")
    assert_bits_equal(qd, q_ref, "q")
    assert (kc_ref.view(torch.uint8) != 0x55).any(), "the append must have written something"


def test_paged_attention_module_over_fp8_cache(fmha, orc):
    """The module carries the static scales: a decode step (quantising append + attention) and a prefill over the same
    quantised cache, against the oracle's chain."""
    from flashck_amd.nn import PagedAttention
    w = gen.workload_appendkv_decode(seed=11, batch=3, hq=8, hk=2, head_dim=128, min_len=20, max_len=400, max_new=3, page_size=64)
    kd, vd = 0.03, 0.025
    k8, v8 = _quantised(w, kd, vd)
    m = PagedAttention(8, 2, 128, rope_mode=2, num_splits=2, k_descale=kd, v_descale=vd)
    assert "k_descale=0.03" in repr(m)
    q, kc, vc = dev(w["q"]), dev(k8), dev(v8)
    o, sl_new = m.decode_step(q, dev(w["knew"]), dev(w["vnew"]), kc, vc, dev(w["seqlen_k"]), dev(w["block_table"]),
                              cu_seqlens_knew=dev(w["cu_seqlens_knew"]), max_seqlen_knew=w["max_new"], rotary_cos=dev(w["rotary_cos"]),
                              rotary_sin=dev(w["rotary_sin"]))
    q_ref, k_ref, v_ref = w["q"].clone(), k8.clone(), v8.clone()
    orc.appendkv(q_ref, k_ref, v_ref, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], cos=w["rotary_cos"], sin=w["rotary_sin"],
                 rope_mode=2, has_mask=True, block_table=w["block_table"], k_descale=kd, v_descale=vd)
    ref_len = w["seqlen_k"] + torch.tensor(w["new"], dtype=torch.int32)
    okw = dict(seqstart_q=w["cu_seqlens_knew"], seqlen_k=ref_len, block_table=w["block_table"], mask_type=2, window=(-1, 0),
               k_descale=kd, v_descale=vd)
    _bytes_equal(kc, k_ref, "k_cache after the step")
    assert torch.equal(sl_new.cpu(), ref_len)
    assert_close(o, orc.fmha_fwd(q_ref, k_ref, v_ref, **okw), 2e-2, "module decode step")
    # prefill of the same (new) tokens as a prompt over the grown cache: same problem through the prefill kernels
    o2 = m.prefill(q, kc, vc, dev(w["cu_seqlens_knew"]), seqlen_k=sl_new, block_table=dev(w["block_table"]), max_seqlen_q=w["max_new"])
    assert_close(o2, orc.fmha_fwd(q_ref, k_ref, v_ref, **okw), 2e-2, "module prefill")
    with pytest.raises(ValueError, match="positive and finite"):
        PagedAttention(8, 2, 128, k_descale=0.0)
