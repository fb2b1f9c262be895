"""Pins the oracle's rotary embedding, appendKV and paged gather with textbook forms and byte-level invariants."""
import numpy as np
import pytest
import torch

from flashck_amd import generators as gen
from helpers import assert_bits_equal


def rope_textbook(x, pos, cos, sin, interleaved):
    """Complex-number form of the rotary embedding in numpy fp32: (a + ib) * (cos + i sin), one IEEE operation at a time."""
    xf = x.float().numpy()
    c = cos.float().numpy()[pos.numpy()][:, None, :]   # [rows, 1, rd/2]
    s = sin.float().numpy()[pos.numpy()][:, None, :]
    rd = cos.shape[1] * 2
    out = xf.copy()
    if interleaved:
        a, b = xf[..., 0:rd:2], xf[..., 1:rd:2]
        out[..., 0:rd:2] = (a * c).astype(np.float32) - (b * s).astype(np.float32)
        out[..., 1:rd:2] = (b * c).astype(np.float32) + (a * s).astype(np.float32)
    else:
        a, b = xf[..., :rd // 2], xf[..., rd // 2:rd]
        out[..., :rd // 2] = (a * c).astype(np.float32) - (b * s).astype(np.float32)
        out[..., rd // 2:rd] = (b * c).astype(np.float32) + (a * s).astype(np.float32)
    return torch.from_numpy(out).to(x.dtype)   # torch rounds to nearest even


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode,rd", [(1, 64), (2, 64), (1, 32), (2, 16)])
def test_rope_matches_textbook_bit_exact(orc, dtype, mode, rd):
    g = torch.Generator().manual_seed(rd + mode)
    x = gen.randn((9, 3, 64), dtype, g)
    cos, sin = gen.rotary_tables(50, rd, dtype)
    pos = torch.tensor([0, 1, 2, 7, 13, 21, 34, 49, 3], dtype=torch.int32)
    got = orc.rope(x, pos, cos, sin, rope_mode=mode)
    assert_bits_equal(got, rope_textbook(x, pos, cos, sin, mode == 1), "rope")
    assert_bits_equal(got[0], x[0], "position 0 is the identity")          # cos 1, sin 0
    assert_bits_equal(got[..., rd:], x[..., rd:], "tail beyond rotary_dim")


def test_rope_preserves_pair_norm(orc):
    # with fp32-exact tables the rotation is orthogonal; in bf16 the pair norms move by rounding only
    g = torch.Generator().manual_seed(2)
    x = gen.randn((4, 2, 128), torch.bfloat16, g)
    cos, sin = gen.rotary_tables(16, 128, torch.bfloat16)
    y = orc.rope(x, torch.tensor([3, 5, 9, 15], dtype=torch.int32), cos, sin, rope_mode=2).float()
    xf = x.float()
    n0 = xf[..., :64] ** 2 + xf[..., 64:] ** 2
    n1 = y[..., :64] ** 2 + y[..., 64:] ** 2
    assert ((n1 - n0).abs() <= 0.03 * n0 + 1e-3).all()


def test_rotary_tables_closed_form():
    cos, sin = gen.rotary_tables(8, 8, torch.float32)
    for p in range(8):
        for i in range(4):
            a = p * 10000.0 ** (-2.0 * i / 8)
            assert abs(float(cos[p, i]) - np.cos(a)) < 1e-6 and abs(float(sin[p, i]) - np.sin(a)) < 1e-6


@pytest.mark.parametrize("page", [16, 128])
@pytest.mark.parametrize("mode", [0, 2])
def test_appendkv_closed_form_and_untouched_bytes(orc, page, mode):
    w = gen.workload_appendkv_decode(seed=60 + page, batch=5, hq=4, hk=2, head_dim=64, min_len=0, max_len=300, max_new=16,
                                     page_size=page)
    q, kc, vc = w["q"].clone(), w["k_cache"].clone(), w["v_cache"].clone()
    orc.appendkv(q, kc, vc, w["knew"], w["vnew"], w["seqlen_k"], w["cu_seqlens_knew"], w["rotary_cos"], w["rotary_sin"],
                 rope_mode=mode, has_mask=True, block_table=w["block_table"])
    touched = torch.zeros(kc.shape[0] * page, dtype=torch.bool)
    cu = w["cu_seqlens_knew"].tolist()
    for b, (L, n) in enumerate(zip(w["lens"], w["new"])):
        pos = torch.arange(L, L + n, dtype=torch.int32)
        want_k = rope_textbook(w["knew"][cu[b]:cu[b + 1]], pos, w["rotary_cos"], w["rotary_sin"], False) if mode else w["knew"][cu[b]:cu[b + 1]]
        want_q = rope_textbook(w["q"][cu[b]:cu[b + 1]], pos, w["rotary_cos"], w["rotary_sin"], False) if mode else w["q"][cu[b]:cu[b + 1]]
        phys = w["block_table"][b, (pos // page).long()].long() * page + (pos % page).long()
        assert_bits_equal(kc.view(-1, 2, 64)[phys], want_k, "appended K rows")
        assert_bits_equal(vc.view(-1, 2, 64)[phys], w["vnew"][cu[b]:cu[b + 1]], "appended V rows")
        assert_bits_equal(q[cu[b]:cu[b + 1]], want_q, "rotated Q rows")
        touched[phys] = True
    # every other byte of the pool is what it was (NaN-filled slots included)
    assert_bits_equal(kc.view(-1, 2, 64)[~touched], w["k_cache"].view(-1, 2, 64)[~touched], "untouched K")
    assert_bits_equal(vc.view(-1, 2, 64)[~touched], w["v_cache"].view(-1, 2, 64)[~touched], "untouched V")


def test_has_mask_false_uses_one_position_for_all_queries(orc):
    g = torch.Generator().manual_seed(9)
    kv = gen.paged_kv([20], 1, 32, torch.float16, g, 16, capacity=[24])
    cos, sin = gen.rotary_tables(32, 32, torch.float16)
    q0 = gen.randn((4, 2, 32), torch.float16, g)
    q = q0.clone()
    orc.appendkv(q, kv["k_cache"], kv["v_cache"], gen.randn((4, 1, 32), torch.float16, g), gen.randn((4, 1, 32), torch.float16, g),
                 kv["seqlen_k"], torch.tensor([0, 4], dtype=torch.int32), cos, sin, rope_mode=1, has_mask=False,
                 block_table=kv["block_table"])
    assert_bits_equal(q, rope_textbook(q0, torch.full((4,), 20, dtype=torch.int32), cos, sin, True), "q at seqlen_k")


def test_paged_gather_round_trip(orc):
    g = torch.Generator().manual_seed(10)
    for page in (1, 16, 128):
        lens = [1, 130, 257]
        kv = gen.paged_kv(lens, 3, 32, torch.bfloat16, g, page)
        for b, n in enumerate(lens):
            got = orc.gather_paged(kv["k_cache"], kv["block_table"][b].contiguous(), n)
            assert_bits_equal(got, kv["k_rows"][b], f"gather page={page}")
