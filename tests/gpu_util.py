"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev_bf16(bits):
    """uint16 bf16 bit patterns (numpy) -> torch.bfloat16 on the GPU, same bytes."""
    t = torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda()
    return t.view(torch.bfloat16)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host_bits(t):
    """torch tensor on the GPU -> numpy; bf16 comes back as uint16 bit patterns."""
    torch.cuda.synchronize()
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    return t.contiguous().cpu().numpy()


def bf16_to_f32(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def ulp_bf16(ref_f32):
    """Size of one bf16 unit in the last place at the magnitude of ref (8 significant bits)."""
    a = np.abs(ref_f32.astype(np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -126)))
    return np.exp2(e - 7)


def check_float_parity(got_f32, ref_f32, what, rel_fro=1e-3, frac_within=0.999):
    """The floating-point bar of this path: relative Frobenius error <= 1e-3 and at least 99.9 % of
    the elements within one bf16 ulp of the reference value."""
    got = got_f32.astype(np.float64)
    ref = ref_f32.astype(np.float64)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    denom = np.linalg.norm(ref)
    err = np.linalg.norm(got - ref) / (denom if denom > 0 else 1.0)
    within = np.abs(got - ref) <= ulp_bf16(ref_f32)
    frac = within.mean()
    assert err <= rel_fro, f"{what}: relative Frobenius error {err:.3e} > {rel_fro}"
    assert frac >= frac_within, f"{what}: only {frac * 100:.3f}% of elements within 1 bf16 ulp"
    return err, frac


# The reference's GELU (oneDNN's gelu_erf minimax polynomial, include/kernels_amx.hpp:242-289) is
# computed as x/2 * (1 + x*P(x^2)).  For pre-activations below about -3.5 the sum 1 + x*P(x^2) cancels
# to 1e-4 .. 1e-7 while its fp32 evaluation keeps an absolute noise of about 2^-24, so there a change of
# the pre-activation by a single fp32 ulp already moves the result by more than one bf16 ulp.  Two
# implementations can only agree to one bf16 ulp in that tail if their fp32 accumulators are
# bit-identical, which no other summation order than AMX's own can provide.
GELU_WELL_CONDITIONED_ABOVE = -3.5


def check_gelu_parity(got_bits, ref_bits, ref_preact, what, frac_all=0.0):
    """bf16 GELU outputs: Frobenius bar on everything, the one-ulp bar on the elements whose reference
    pre-activation is above GELU_WELL_CONDITIONED_ABOVE; the fraction over all elements is returned
    (and must reach frac_all)."""
    got, ref = bf16_to_f32(got_bits), bf16_to_f32(ref_bits)
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    err = np.linalg.norm(got.astype(np.float64) - ref) / np.linalg.norm(ref.astype(np.float64))
    assert err <= 1e-3, f"{what}: relative Frobenius error {err:.3e}"
    within = np.abs(got.astype(np.float64) - ref) <= ulp_bf16(ref)
    good = ref_preact > GELU_WELL_CONDITIONED_ABOVE
    frac_good = within[good].mean()
    frac = within.mean()
    assert frac_good >= 0.999, f"{what}: {frac_good * 100:.3f}% within 1 bf16 ulp where GELU is well conditioned"
    assert frac >= frac_all, f"{what}: {frac * 100:.3f}% within 1 bf16 ulp over all elements"
    return err, frac_good, frac
