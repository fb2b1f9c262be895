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
