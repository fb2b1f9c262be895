"""GPU parity: LSE combine kernel against the CPU oracle and closed forms."""
import pytest
import torch

from helpers import assert_bits_equal, assert_close, dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ns", [1, 2, 5, 8, 16, 33])
@pytest.mark.parametrize("dv", [64, 128, 256])
def test_combine_matches_oracle(fmha, orc, dtype, ns, dv):
    g = torch.Generator().manual_seed(ns * 1000 + dv)
    B, H, S = 2, 3, 5
    o_acc = torch.randn(B, H, ns, S, dv, generator=g)
    lse = torch.randn(B, H, ns, S, generator=g) * 3
    # empty splits and one row without any visible key
    lse[0, 0, ns // 2, :] = float("-inf")
    lse[1, 2, :, 3] = float("-inf")
    o = fmha.fmha_fwd_splitkv_combine(dev(lse), dev(o_acc), dtype)
    ref = orc.splitkv_combine(lse, o_acc, dtype)
    assert_close(o, ref, 1e-2 if dtype == torch.float16 else 2e-2, "combine")
    assert (o[1, 3, 2].float() == 0).all(), "a row with no visible key must come out as zeros"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_single_split_is_a_cast(fmha, dtype):
    g = torch.Generator().manual_seed(1)
    o_acc = torch.randn(2, 4, 1, 3, 128, generator=g)
    lse = torch.randn(2, 4, 1, 3, generator=g)
    o = fmha.fmha_fwd_splitkv_combine(dev(lse), dev(o_acc), dtype)
    assert_bits_equal(o, o_acc[:, :, 0].permute(0, 2, 1, 3).contiguous().to(dtype), "ns=1")


def test_group_mode_layout(fmha, orc):
    g = torch.Generator().manual_seed(2)
    cu = torch.tensor([0, 3, 4, 9], dtype=torch.int32)
    o_acc = torch.randn(1, 4, 3, 9, 64, generator=g)
    lse = torch.randn(1, 4, 3, 9, generator=g)
    o = fmha.fmha_fwd_splitkv_combine(dev(lse), dev(o_acc), torch.bfloat16, cu_seqlens_q=dev(cu), max_seqlen_q=5)
    ref = orc.splitkv_combine(lse, o_acc, torch.bfloat16, seqstart_q=cu)
    assert_close(o, ref, 2e-2, "group combine")


@pytest.mark.parametrize("dv,rows", [(64, 170), (128, 90), (256, 45)])
def test_combine_many_rows(fmha, orc, dv, rows):
    """Enough output rows that the launcher takes 256-thread workgroups (small problems run one wave per workgroup):
    both workgroup shapes, incl. a last workgroup that is only partly filled."""
    g = torch.Generator().manual_seed(dv + rows)
    B, H, ns = 3, 33, 3
    o_acc = torch.randn(B, H, ns, rows, dv, generator=g)
    lse = torch.randn(B, H, ns, rows, generator=g) * 2
    lse[2, 5, 1, :] = float("-inf")
    o = fmha.fmha_fwd_splitkv_combine(dev(lse), dev(o_acc), torch.bfloat16)
    ref = orc.splitkv_combine(lse, o_acc, torch.bfloat16)
    assert_close(o, ref, 2e-2, "combine, many rows")
