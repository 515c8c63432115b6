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
