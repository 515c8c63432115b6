"""Shared helpers of the GPU parity tests: seeded inputs, numpy<->torch views, tolerances."""
import numpy as np

import oracle

# tolerances stated by the task: fp32/fp64 max|d| <= 1e-5*K*max|A|*max|B|;
# fp16/bf16 <= 2e-2 relative, normalised by max|C_ref|
def float_tol(k, a, b):
    return 1e-5 * max(k, 1) * float(np.abs(a).max(initial=0.0)) * float(np.abs(b).max(initial=0.0))


HALF_REL = 2e-2


def np_dtype_code(arr, bf16=False):
    return oracle.BF16 if bf16 else oracle.dtype_code(arr)


def randn(rng, shape, dtype, scale=1.0):
    """N(0,1)*scale in `dtype`; 'bf16' gives uint16 bit patterns."""
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    if dtype == "bf16":
        return oracle.to_bf16_bits(x)
    return x.astype(dtype)


def to_f64(arr, bf16=False):
    if bf16:
        return oracle.from_bf16_bits(arr).astype(np.float64)
    return arr.astype(np.float64)


def to_torch(arr, device, bf16=False):
    import torch
    if bf16:
        return torch.from_numpy(arr.view(np.int16)).to(device).view(torch.bfloat16)
    if arr.dtype == np.uint16 or arr.dtype == np.uint32 or arr.dtype == np.uint64:
        raise ValueError("torch has no matching unsigned dtype")
    return torch.from_numpy(arr).to(device)


def from_torch(t):
    import torch
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


# ---- one-rounding check of 16-bit results ------------------------------------------------------------------------
# A 16-bit product that accumulates in float32 over all of K and rounds once differs from RNE(exact result) only where the
# exact result lies closer to a rounding boundary (the midpoint of two neighbouring 16-bit values) than the float32
# accumulation error.  Products of two 16-bit values are exact in float32 and float64, and a float64 sum over K <= 2^20
# terms is exact to ~2^-33 of the sum of magnitudes, so `ref64` stands for the exact result.
_SIG_BITS = {"bf16": 8, "f16": 11}


def rne16(ref64, fmt):
    """(rounded value, ulp, distance of ref64 from the nearest rounding boundary) in float64, round-to-nearest-even."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    _, e = np.frexp(ref64)                       # |x| = f * 2^e, f in [0.5, 1)
    if fmt == "f16":
        e = np.maximum(e, -13)                   # subnormal halves share the ulp of the smallest normal binade
    ulp = np.ldexp(1.0, e - _SIG_BITS[fmt])
    q = ref64 / ulp                              # exact: a power-of-two scaling
    r = np.rint(q)                               # ties to even
    dist = np.abs(q - (np.floor(q) + 0.5)) * ulp
    return r * ulp, ulp, dist


def assert_one_rounding(got64, ref64, spread64, k, fmt, what="", min_exact=0.75):
    """got64: the 16-bit results widened to float64; ref64: the exact result (float64 GEMM + C0); spread64: the size of
    the partial sums on the way, |C0| + sqrt(A^2 . B^2) (one standard deviation of a sum of k products of random sign).
    Every element must be within one 16-bit ulp (plus the accumulation bound below) of RNE(ref64), and bit-equal to it wherever ref64 is further from a
    rounding boundary than  8 sqrt(k + 2) 2^-24 (|ref64| + 4 spread64): each of the k float32 roundings errs by at most
    2^-24 of a partial sum, partial sums stay below |ref| + 4 spread, and independent errors add up like sqrt(k) -- the
    factor 8 leaves two orders of magnitude above the expected error, whatever the order of summation."""
    want, ulp, dist = rne16(ref64, fmt)
    err = np.abs(np.asarray(got64, np.float64) - want)
    bound = 8.0 * np.sqrt(k + 2.0) * 2.0 ** -24 * (np.abs(ref64) + 4.0 * np.asarray(spread64, np.float64))
    # (results that cancel to nearly nothing have ulps below the accumulation error itself: the bound is allowed on top;
    #  1.5 ulp admits one step on the 16-bit grid, also across a binade boundary)
    far = err > 1.5 * ulp + bound
    assert not far.any(), f"{what}: {int(far.sum())} elements differ from RNE(exact) by more than one ulp (max {float((err / ulp).max())} ulp)"
    clear = dist > bound
    assert clear.mean() >= min_exact, f"{what}: only {clear.mean():.4f} of the elements are clear of a rounding boundary"
    bad = clear & (err != 0)
    assert not bad.any(), f"{what}: {int(bad.sum())} elements away from any rounding boundary are not RNE(exact)"
