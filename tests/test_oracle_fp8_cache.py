"""CPU: pins of the oracle's fp32 -> e4m3 conversion and of its appendKV into a quantised cache."""
import math

import pytest
import torch

from flashck_amd import generators as gen


def _all_16bit_values(dtype):
    x = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(dtype).float()
    return x[torch.isfinite(x)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_f32_to_fp8_on_every_16bit_value(orc, dtype):
    """Every finite bf16 / fp16 value: inside +-448 the byte torch's round-to-nearest-even cast gives, beyond it the
    largest finite code of that sign (torch's cast does not saturate, it gives NaN there)."""
    x = _all_16bit_values(dtype)
    got = torch.tensor([orc.f32_to_fp8(v) for v in x.tolist()], dtype=torch.uint8)
    inside = x.abs() <= 448
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(got[inside], ref[inside])
    want = torch.where(x[~inside] > 0, 0x7e, 0xfe).to(torch.uint8)
    assert torch.equal(got[~inside], want)


def test_f32_to_fp8_ties_subnormals_specials(orc):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(50000, generator=g) * torch.exp(torch.randn(50000, generator=g) * 4)).float()
    x = x[x.abs() <= 448]
    got = torch.tensor([orc.f32_to_fp8(v) for v in x.tolist()], dtype=torch.uint8)
    assert torch.equal(got, x.to(torch.float8_e4m3fn).view(torch.uint8))
    # halfway cases between neighbouring codes go to the even code; the subnormal grid is 2^-9
    for value, byte in [(2.0 ** -10, 0x00), (3 * 2.0 ** -10, 0x02), (2.0 ** -9, 0x01), (1.0625, 0x38), (1.1875, 0x3a), (448.0, 0x7e),
                        (463.9, 0x7e), (1e30, 0x7e), (-1e30, 0xfe), (0.0, 0x00), (-0.0, 0x80)]:
        assert orc.f32_to_fp8(value) == byte, value
    assert orc.f32_to_fp8(float("nan")) & 0x7f == 0x7f
    assert orc.f32_to_fp8(float("inf")) == 0x7f and orc.f32_to_fp8(float("-inf")) == 0xff
    # decode(encode(x)) is the identity on the 254 non-NaN codes
    for b in range(256):
        if b & 0x7f != 0x7f:
            assert orc.f32_to_fp8(orc.fp8_to_f32(b)) == b


@pytest.mark.parametrize("dtype,rope_mode", [(torch.bfloat16, 2), (torch.float16, 1), (torch.bfloat16, 0)])
def test_appendkv_into_fp8_cache_is_the_quantised_16bit_append(orc, dtype, rope_mode):
    """cache8 == fp8(cache16 / descale) on the appended rows, where cache16 is what the (already pinned) 16-bit append
    writes; every other byte of the pool is untouched; q is rotated as in the 16-bit path."""
    w = gen.workload_appendkv_decode(seed=77, batch=3, hq=4, hk=2, head_dim=64, min_len=5, max_len=90, max_new=6, page_size=16, dtype=dtype)
    kd, vd = 0.02, 0.05
    kw = dict(cos=w["rotary_cos"], sin=w["rotary_sin"], rope_mode=rope_mode, has_mask=True, block_table=w["block_table"])
    q16, k16, v16 = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    orc.appendkv(q16, k16, v16, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], **kw)
    fill = torch.full(w["k_cache"].shape, 0x55, dtype=torch.uint8)
    q8, k8, v8 = w["q"].clone(), fill.clone().view(torch.float8_e4m3fn), fill.clone().view(torch.float8_e4m3fn)
    orc.appendkv(q8, k8, v8, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], k_descale=kd, v_descale=vd, **kw)
    assert torch.equal(q8.view(torch.int16), q16.view(torch.int16))
    written = torch.zeros(w["k_cache"].shape[:2], dtype=torch.bool)
    page = w["k_cache"].shape[1]
    for b, (L, n) in enumerate(zip(w["seqlen_k"].tolist(), w["new"])):
        for t in range(L, L + n):
            written[w["block_table"][b, t // page], t % page] = True
    want_k = (k16.float() / kd).to(torch.float8_e4m3fn).view(torch.uint8)
    want_v = (v16.float() / vd).to(torch.float8_e4m3fn).view(torch.uint8)
    k8b, v8b = k8.view(torch.uint8), v8.view(torch.uint8)
    assert written.sum().item() == sum(w["new"])
    assert torch.equal(k8b[written], want_k[written]) and torch.equal(v8b[written], want_v[written])
    assert (k8b[~written] == 0x55).all() and (v8b[~written] == 0x55).all()


def test_appendkv_fp8_saturates(orc):
    """Values beyond 448 * descale land on +-448 instead of overflowing."""
    w = gen.workload_appendkv_decode(seed=78, batch=1, hq=2, hk=1, head_dim=64, min_len=3, max_len=3, max_new=1, page_size=16)
    w["knew"][:] = 30.0
    w["vnew"][:] = -30.0
    k8 = torch.zeros(w["k_cache"].shape, dtype=torch.uint8).view(torch.float8_e4m3fn)
    v8 = k8.clone()
    orc.appendkv(None, k8, v8, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], block_table=w["block_table"],
                 k_descale=0.01, v_descale=0.01)
    L = int(w["seqlen_k"][0])
    page = int(w["block_table"][0, L // 16])
    assert (k8.view(torch.uint8)[page, L % 16] == 0x7e).all() and (v8.view(torch.uint8)[page, L % 16] == 0xfe).all()
