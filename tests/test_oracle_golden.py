"""The CPU oracle against golden vectors produced by ck_tile's own host reference functions
(tests/golden/ck_tile_host_golden.cpp): rotary embedding and the gemm -> mask -> softmax -> gemm attention chain."""
import pytest
import torch

from golden import reader
from helpers import assert_bits_equal

G = reader.load()


@pytest.mark.parametrize("tag,mode", [("rope_half_bf16", 2), ("rope_inter_bf16", 1), ("rope_half_fp16_partial", 2),
                                      ("rope_inter_fp16_partial", 1)])
def test_rope_bit_exact(orc, tag, mode):
    x, cos, sin, y = (G[f"{tag}.{k}"] for k in ("x", "cos", "sin", "y"))   # x, y: [heads, seq, d]
    seq = x.shape[1]
    got = orc.rope(x.transpose(0, 1).contiguous(), torch.arange(seq, dtype=torch.int32), cos, sin, rope_mode=mode)
    assert_bits_equal(got.transpose(0, 1), y, tag)


ATTN = ["attn_bf16_nomask", "attn_bf16_causal_br", "attn_bf16_causal_tl", "attn_bf16_window_br", "attn_bf16_causal_sq_gt_sk",
        "attn_fp16_nomask", "attn_fp16_window_tl", "attn_bf16_d40_dv72_causal_br", "attn_fp16_d192_dv128_nomask"]


@pytest.mark.parametrize("tag", ATTN)
def test_attention_chain_bit_exact(orc, tag):
    q, k, vt, o, lse = (G[f"{tag}.{n}"] for n in ("q", "k", "vt", "o", "lse"))   # q [bh, sq, d], vt [bh, dv, sk]
    mask_type, wl, wr, _ = G[f"{tag}.mask"].tolist()
    scale = float(G[f"{tag}.scale"][0])
    got, got_lse = orc.fmha_fwd(q.unsqueeze(2).contiguous(), k.unsqueeze(2).contiguous(),
                                vt.transpose(1, 2).unsqueeze(2).contiguous(), return_lse=True, scale=scale,
                                mask_type=mask_type, window=(wl, wr))
    assert_bits_equal(got.squeeze(2), o, tag + " o")
    # rows without a visible key: the host reference stores max + ln(0) with max reset to 0, i.e. -inf
    assert torch.equal(torch.isinf(got_lse[:, 0]), torch.isinf(lse))
    fin = torch.isfinite(lse)
    assert (got_lse[:, 0][fin] - lse[fin]).abs().max() <= 1e-6


@pytest.mark.parametrize("tag", ATTN)
def test_mask_matches_golden_probabilities(orc, tag):
    # p == 0 in the golden probabilities exactly where the oracle's visibility predicate says "masked"
    p = G[f"{tag}.p"].float()
    mask_type, wl, wr, _ = G[f"{tag}.mask"].tolist()
    _, sq, sk = p.shape
    vis = torch.tensor([[orc.visible(mask_type, (wl, wr), sq, sk, i, j) for j in range(sk)] for i in range(sq)])
    full_rows = vis.any(dim=1)
    assert ((p[0] > 0) == vis)[full_rows].all()
