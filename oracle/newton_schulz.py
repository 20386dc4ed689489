"""Oracle for the quintic Newton-Schulz orthogonalisation (test infrastructure only).

Follows, op for op and rounding for rounding:
  * `zeropower_via_newtonschulz5(G, epsilon)`   -- reference dion/muon.py:620-647
    (identical twin in dion/newton_schulz_triton.py:305-333): per-iteration
    coefficient schedule, batched, transpose-to-wide, Frobenius pre-normalisation.
  * `zeropower_via_newtonschulz5(G, steps, eps)` -- reference dion/muon_reference.py:10-27:
    fixed Keller coefficients, 2-D only, normalisation before the transpose.
"""
import torch

# reference dion/muon.py:625-631
NS_SCHEDULE_COEFFS = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
# reference dion/muon_reference.py:16
NS_KELLER_COEFFS = (3.4445, -4.7750, 2.0315)


def ns5(G, epsilon=1e-7, coeffs=NS_SCHEDULE_COEFFS, compute_dtype=torch.bfloat16):
    """reference dion/muon.py:633-647, with the working dtype made a parameter.

    `compute_dtype=torch.bfloat16` is the reference path (every `@`, scalar
    multiply and add rounds to bf16).  float32 / float64 evaluate the same
    recurrence without the intermediate roundings.
    """
    X = G.to(dtype=compute_dtype)
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    X = X / (X.norm(dim=(-2, -1), keepdim=True) + epsilon)
    for a, b, c in coeffs:
        A = X @ X.mT
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    if tall:
        X = X.mT
    return X


def ns5_keller(G, steps=5, eps=1e-7, compute_dtype=torch.bfloat16):
    """reference dion/muon_reference.py:10-27 (fixed coefficients, 2-D only)."""
    assert G.ndim == 2, "Expected 2D tensor"
    a, b, c = NS_KELLER_COEFFS
    X = G.to(compute_dtype)
    X = X / (X.norm() + eps)
    if G.size(0) > G.size(1):
        X = X.T
    for _ in range(steps):
        A = X @ X.T
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    if G.size(0) > G.size(1):
        X = X.T
    return X


def ns5_closed_form(G, coeffs=NS_SCHEDULE_COEFFS, epsilon=1e-7):
    """What the mathematics fixes: with G = U diag(s) V^T the iteration maps
    s -> p_k(...p_1(s / (||G||_F + eps))) with p(x) = a x + b x^3 + c x^5 and
    leaves U, V untouched.  Evaluated in float64; independent of any matmul
    ordering, transposition or operand layout in `ns5`.
    """
    G64 = G.to(torch.float64)
    U, s, Vh = torch.linalg.svd(G64, full_matrices=False)
    s = s / (torch.linalg.matrix_norm(G64, keepdim=True).squeeze(-1) + epsilon)
    for a, b, c in coeffs:
        s = a * s + b * s**3 + c * s**5
    return U @ torch.diag_embed(s) @ Vh


def ns_flops(m, n, steps=5, symmetric=False):
    """FLOP conventions.  Dense (reference benchmark/benchmark_newton_shultz.py:33-42):
    per iteration 4 m_w^2 n_w + 2 m_w^3.  Symmetric-output execution: 3 m_w^2 n_w + m_w^3.
    """
    mw, nw = min(m, n), max(m, n)
    per = (3 * mw * mw * nw + mw**3) if symmetric else (4 * mw * mw * nw + 2 * mw**3)
    return steps * per
