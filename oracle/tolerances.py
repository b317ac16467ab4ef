"""Error bounds of the attention parity checks (test infrastructure, like the rest of oracle/).

The absolute bound of 2e-2 on bf16 outputs says nothing when the outputs themselves are small
(Q, K, V ~ N(0,1)/sqrt(128) gives max|ref| ~ 5e-3: an all-zero output would pass), so every check
is scaled by the magnitude of the oracle's result as well:

    max|out - ref| <= max(2e-2 * max|ref|, 2 bf16 ulp of max|ref|)   and   <= abs_tol (2e-2)
"""
from __future__ import annotations

import math

import torch

ABS_TOL_BF16 = 2e-2    # max-abs bound of bf16 attention outputs
REL_TOL_BF16 = 2e-2    # the same bound relative to the largest reference value
REL_TOL_FP32 = 1e-3    # partial results (fp32 accumulation), before the rounding of the output to bf16


def bf16_ulp(x: float) -> float:
    """Spacing of bf16 numbers at magnitude x (8 significant bits)."""
    if x <= 0.0 or not math.isfinite(x):
        return 0.0
    return 2.0 ** (math.floor(math.log2(x)) - 7)


def attn_bound(ref: torch.Tensor, abs_tol: float = ABS_TOL_BF16, rel_tol: float = REL_TOL_BF16) -> float:
    m = float(ref.abs().max())
    return min(abs_tol, max(rel_tol * m, 2.0 * bf16_ulp(m)))


def assert_attn_close(out: torch.Tensor, ref: torch.Tensor, what: str = "", abs_tol: float = ABS_TOL_BF16,
                      rel_tol: float = REL_TOL_BF16) -> float:
    """out, ref: float tensors on the CPU.  Returns the measured max-abs error."""
    assert out.shape == ref.shape, f"{what}: shape {tuple(out.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    err = float((out - ref).abs().max())
    bound = attn_bound(ref, abs_tol, rel_tol)
    assert err <= bound, f"{what}: max abs err {err:.3e} > bound {bound:.3e} (max|ref| {float(ref.abs().max()):.3e})"
    return err
