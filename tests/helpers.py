"""Shared helpers of the parity tests."""
import torch

# Tolerances of the parity tests: max-abs error of attention outputs against the fp32-accumulated reference
ATOL = {torch.float16: 1e-2, torch.bfloat16: 2e-2}


# where the parity tests put their tensors (the emulator run of these tests sets it to "cpu")
DEVICE = "cuda"


def dev(x, device="cuda"):
    if isinstance(x, torch.Tensor):
        return x.to(device)
    return x


def bits(t):
    """Bit pattern of a 16-bit float tensor (NaN-safe equality)."""
    return t.contiguous().view(torch.int16).cpu()


def assert_bits_equal(a, b, what=""):
    ba, bb = bits(a), bits(b)
    assert ba.shape == bb.shape, f"{what}: shape {ba.shape} vs {bb.shape}"
    bad = (ba != bb).nonzero()
    assert bad.numel() == 0, f"{what}: {bad.shape[0]} of {ba.numel()} elements differ, first at {bad[0].tolist()}"


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def assert_close(a, b, atol, what=""):
    a, b = a.float().cpu(), b.float().cpu()
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    assert torch.isfinite(a).all(), f"{what}: non-finite values in the result"
    err = (a - b).abs().max().item()
    assert err <= atol, f"{what}: max-abs error {err:.3e} > {atol:.1e}"


def assert_lse_close(a, b, atol=2e-3, what=""):
    a, b = a.float().cpu(), b.float().cpu()
    inf_a, inf_b = torch.isinf(a) & (a < 0), torch.isinf(b) & (b < 0)
    assert torch.equal(inf_a, inf_b), f"{what}: -inf pattern differs"
    fin = ~inf_a
    if fin.any():
        err = (a[fin] - b[fin]).abs().max().item()
        assert err <= atol, f"{what}: max-abs LSE error {err:.3e} > {atol:.1e}"


# e4m3 outputs of the all-fp8 roles.  The kernels cast the probabilities relative to the running row maximum (as ck_tile's
# device pipeline does), the oracle casts the normalised ones (as ck_tile's host reference does; small probabilities
# then fall into e4m3's subnormal range, which makes that order the noisier of the two).  The two agree up to the noise
# of that cast: a result may land one e4m3 rounding point away, and where a sum of terms of mixed sign nearly cancels
# only an absolute bound holds.  One rounding point and 0.0625 (for values of unit scale) is also what ck_tile's own fp8
# check allows.  A cast error of up to 2^-4 per probability on top of the output's own rounding can carry a rare value
# further: `outliers` is the fraction allowed beyond (one step, atol); nothing may be beyond twice that.
FP8_ATOL = 0.0625


def fp8_step(x):
    """spacing of e4m3 values at the magnitude of x"""
    return torch.exp2(torch.floor(torch.log2(x.abs().clamp(min=2.0 ** -6))) - 3)


def assert_fp8_close(a, b, what="", atol=FP8_ATOL, outliers=0.0):
    """a: e4m3 result; b: e4m3 or wider reference."""
    assert a.dtype == torch.float8_e4m3fn, f"{what}: result is {a.dtype}"
    a, b = a.cpu().float(), b.cpu().float()   # e4m3 is widened on the host
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    assert torch.isfinite(a).all(), f"{what}: non-finite values in the result"
    diff = (a - b).abs()
    bound = torch.maximum(fp8_step(torch.maximum(a.abs(), b.abs())), torch.tensor(float(atol)))
    far = int((diff > 2 * bound).sum())
    assert far == 0, f"{what}: {far} of {a.numel()} values are more than two e4m3 steps and {2 * atol} apart, worst {diff.max().item():.3f}"
    out = int((diff > bound).sum())
    assert out <= outliers * a.numel(), (f"{what}: {out} of {a.numel()} values are more than one e4m3 step and {atol} apart "
                                         f"(allowed: {outliers:g} of them), worst {diff.max().item():.3f}")


def assert_fp8_roles_close(o, oracle8, fine, what="", atol=FP8_ATOL):
    """o: e4m3 result of the all-fp8 roles; oracle8: the oracle with the same roles (probabilities cast in the host
    reference's order); fine: the oracle on the same e4m3 inputs with 16-bit roles for Q, P and O (times o_scale)."""
    assert_fp8_close(o, fine, what + " vs the 16-bit roles", atol, outliers=1e-4)
    assert_fp8_close(o, oracle8, what + " vs the fp8 roles of the oracle", atol, outliers=1e-3)
    f = fine.cpu().float()
    e_dev, e_orc = (o.cpu().float() - f).abs().mean().item(), (oracle8.cpu().float() - f).abs().mean().item()
    assert e_dev <= 1.05 * e_orc + 1e-6, f"{what}: mean error to the 16-bit roles {e_dev:.5f}, the oracle's fp8 roles have {e_orc:.5f}"
