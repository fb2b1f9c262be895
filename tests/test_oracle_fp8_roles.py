"""CPU: the oracle's all-fp8 roles (Q, K, V, P and O in e4m3; FmhaFwdTypeConfig<fp8_t>,
core/module/kernels/attention_kernels/fmha_common_jinja.h:157-171) pinned against an independent restatement with
torch's float8_e4m3fn casts and against closed forms that a dropped P rounding, a dropped output scale or a missing
saturation would fail."""
import math

import torch

F8 = torch.float8_e4m3fn


def _q8(x, s):
    return (x / s).clamp(-448, 448).to(F8)


def _torch_fp8_attention(q8, k8, v8, scale, kd, vd, o_scale, causal):
    """Host-reference order of operations: softmax in fp32, P cast to e4m3, second product in fp32, saturating cast."""
    B, sq, Hq, D = q8.shape
    sk, Hk = k8.shape[1], k8.shape[2]
    qf = q8.float()
    kf = (k8.float() * kd).repeat_interleave(Hq // Hk, 2)
    vf = (v8.float() * vd).repeat_interleave(Hq // Hk, 2)
    s = torch.einsum("bqhd,bkhd->bhqk", qf, kf) * scale
    if causal:
        s = s.masked_fill(~torch.ones(sq, sk).tril(sk - sq).bool(), float("-inf"))
    p8 = s.softmax(-1).to(F8).float()
    o = torch.einsum("bhqk,bkhd->bqhd", p8, vf) * o_scale
    return o.clamp(-448, 448).to(F8)


def _codes(t):
    """e4m3 bytes as integers that are monotonic in the value (sign-magnitude -> signed)."""
    u = t.view(torch.uint8).to(torch.int32)
    return torch.where(u >= 128, -(u - 128), u)


def test_fp8_roles_against_torch_restatement(orc):
    g = torch.Generator().manual_seed(5)
    B, sq, sk, Hq, Hk, D = 2, 37, 90, 4, 2, 64
    qs, kd, vd = 0.02, 0.025, 0.03
    Q = _q8(torch.randn(B, sq, Hq, D, generator=g), qs)
    K = _q8(torch.randn(B, sk, Hk, D, generator=g), kd)
    V = _q8(torch.randn(B, sk, Hk, D, generator=g), vd)
    scale = qs / math.sqrt(D)
    for causal, o_scale in ((False, 1.0), (True, 1.0), (True, 24.0)):
        kw = dict(mask_type=2, window=(-1, 0)) if causal else {}
        o = orc.fmha_fwd(Q, K, V, scale=scale, k_descale=kd, v_descale=vd, o_scale=o_scale, **kw)
        assert o.dtype == F8
        ref = _torch_fp8_attention(Q, K, V, scale, kd, vd, o_scale, causal)
        diff = (_codes(o) - _codes(ref)).abs()
        # the two differ in the order of fp32 additions only: a value may land on the other side of a rounding point
        assert diff.max().item() <= 1, f"causal={causal} o_scale={o_scale}: codes differ by {diff.max().item()}"
        assert (diff == 0).float().mean().item() > 0.99, f"causal={causal} o_scale={o_scale}: {(diff != 0).sum().item()} codes differ"


def _two_key_case(d=64):
    """q = e0, keys 0 and -1.25 * e0, values 0 and 416, scale 1: scores (0, -1.25).
    Normalised P = (0.7773, 0.2227); e4m3(0.2227) = 14/64 = 0.21875, so O = 0.21875 * 416 = 91 -> 88 (grid 80, 88, 96);
    without the cast of P it would be 0.2227 * 416 = 92.6 -> 96."""
    q = torch.zeros(1, 1, 1, d)
    q[..., 0] = 1.0
    k = torch.zeros(1, 2, 1, d)
    k[0, 1, 0, 0] = -1.25
    v = torch.zeros(1, 2, 1, d)
    v[0, 1] = 416.0
    return q.to(F8), k.to(F8), v.to(F8)


def test_p_is_cast_to_e4m3_before_the_second_product(orc):
    q, k, v = _two_key_case()
    o = orc.fmha_fwd(q, k, v, scale=1.0)
    assert torch.all(o.float() == 88.0), o.float().unique()
    # the same through the split path when one split holds both keys; the combine writes e4m3
    o_acc, lse_acc = orc.fmha_splitkv(q, k, v, 1, scale=1.0)
    o1 = orc.splitkv_combine(lse_acc, o_acc, F8)
    assert torch.all(o1.float() == 88.0), o1.float().unique()
    # one key per split: P = 1 inside each split and the merge weights are fp32, never cast: 0.2227 * 416 = 92.6 -> 96
    o_acc, lse_acc = orc.fmha_splitkv(q, k, v, 2, scale=1.0)
    o2 = orc.splitkv_combine(lse_acc, o_acc, F8)
    assert torch.all(o2.float() == 96.0), o2.float().unique()


def test_output_scale_and_saturation(orc):
    """One key: P = 1, O = v_descale * v * o_scale.  3 * 0.5 * 16 = 24 is a grid value; 3 * 0.5 * 512 = 768 saturates at 448,
    with the sign kept."""
    d = 64
    q = torch.ones(1, 1, 1, d).to(F8)
    k = torch.ones(1, 1, 1, d).to(F8)
    v = torch.full((1, 1, 1, d), 3.0)
    v[..., 1::2] = -3.0
    v = v.to(F8)
    o = orc.fmha_fwd(q, k, v, scale=0.1, v_descale=0.5, o_scale=16.0).float()
    assert torch.all(o[..., 0::2] == 24.0) and torch.all(o[..., 1::2] == -24.0)
    o = orc.fmha_fwd(q, k, v, scale=0.1, v_descale=0.5, o_scale=512.0).float()
    assert torch.all(o[..., 0::2] == 448.0) and torch.all(o[..., 1::2] == -448.0)


def test_k_descale_multiplies_the_scores(orc):
    """Two keys whose scores differ by k_descale * 8: with k_descale = 0.25 the weights are (1, e^-2) / (1 + e^-2)."""
    d = 64
    q = torch.zeros(1, 1, 1, d)
    q[..., 0] = 1.0
    k = torch.zeros(1, 2, 1, d)
    k[0, 1, 0, 0] = -8.0
    v = torch.zeros(1, 2, 1, d)
    v[0, 0] = 64.0
    q, k, v = q.to(F8), k.to(F8), v.to(F8)
    o = orc.fmha_fwd(q, k, v, scale=1.0, k_descale=0.25).float()
    w0 = 1.0 / (1.0 + math.exp(-2.0))                      # 0.8808 -> e4m3 0.875
    expect = torch.tensor(0.875 * 64.0).to(F8).float()     # 56
    assert abs(w0 - 0.875) < 1 / 32 and torch.all(o == expect), o.unique()


def test_one_split_combine_equals_the_forward(orc):
    g = torch.Generator().manual_seed(6)
    B, sq, sk, Hq, Hk, D = 2, 3, 70, 4, 2, 64
    Q = _q8(torch.randn(B, sq, Hq, D, generator=g), 0.02)
    K = _q8(torch.randn(B, sk, Hk, D, generator=g), 0.02)
    V = _q8(torch.randn(B, sk, Hk, D, generator=g), 0.02)
    kw = dict(scale=0.02 / 8, k_descale=0.02, v_descale=0.02, mask_type=2, window=(-1, 0))
    o = orc.fmha_fwd(Q, K, V, **kw)
    o_acc, lse_acc = orc.fmha_splitkv(Q, K, V, 1, **kw)
    o1 = orc.splitkv_combine(lse_acc, o_acc, F8)
    assert torch.equal(o.view(torch.uint8), o1.view(torch.uint8))


def test_elementwise_bias_is_float32(orc):
    """BiasDataType of the fp8 roles is float: against the torch restatement with the bias added to the scores, for a
    bias shared by all heads and batches, per head, and per batch and head."""
    g = torch.Generator().manual_seed(8)
    B, sq, sk, Hq, Hk, D = 2, 9, 40, 4, 2, 64
    qs, kd, vd = 0.02, 0.025, 0.03
    Q = _q8(torch.randn(B, sq, Hq, D, generator=g), qs)
    K = _q8(torch.randn(B, sk, Hk, D, generator=g), kd)
    V = _q8(torch.randn(B, sk, Hk, D, generator=g), vd)
    scale = qs / math.sqrt(D)
    for shape in ((1, 1, sq, sk), (1, Hq, sq, sk), (B, Hq, sq, sk + 2)):
        bias = (torch.randn(*shape, generator=g) * 2).contiguous()
        o = orc.fmha_fwd(Q, K, V, scale=scale, k_descale=kd, v_descale=vd, bias=bias)
        qf = Q.float()
        kf = (K.float() * kd).repeat_interleave(Hq // Hk, 2)
        vf = (V.float() * vd).repeat_interleave(Hq // Hk, 2)
        s_ = torch.einsum("bqhd,bkhd->bhqk", qf, kf) * scale + bias[..., :sk]
        ref = torch.einsum("bhqk,bkhd->bqhd", s_.softmax(-1).to(F8).float(), vf).clamp(-448, 448).to(F8)
        diff = (_codes(o) - _codes(ref)).abs()
        assert diff.max().item() <= 1 and (diff == 0).float().mean().item() > 0.99, f"bias {shape}: {(diff != 0).sum().item()} codes differ"
    # a bias in another type is refused by the wrapper
    import pytest
    with pytest.raises(AssertionError):
        orc.fmha_fwd(Q, K, V, scale=scale, bias=torch.zeros(1, 1, sq, sk).to(F8))
