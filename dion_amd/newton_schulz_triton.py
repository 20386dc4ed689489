"""Import-path twin of reference dion/newton_schulz_triton.py: the same four public names, on the HIP kernels.

`newton_schulz_triton` keeps the fused-epilogue rounding of the reference's Triton path (only A, B and X are
rounded to bf16: dion/newton_schulz_triton.py:336-374); `zeropower_via_newtonschulz5` keeps the eager op-by-op
rounding (dion/newton_schulz_triton.py:305-333).
"""
from torch import Tensor

from .newton_schulz import NS_SCHEDULE_COEFFS, newton_schulz, ns_line_1, ns_line_2, zeropower_via_newtonschulz5

__all__ = ["ns_line_1", "ns_line_2", "newton_schulz_triton", "zeropower_via_newtonschulz5"]


def newton_schulz_triton(G: Tensor, epsilon: float = 1e-7) -> Tensor:
    return newton_schulz(G, epsilon=epsilon, coeffs=NS_SCHEDULE_COEFFS, faithful=False)
