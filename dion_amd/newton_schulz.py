"""Newton-Schulz orthogonalisation on the MI355X kernels.

Mirrors the reference operator interface:
  * `zeropower_via_newtonschulz5(G, epsilon=1e-7)`           -- reference dion/muon.py:620-647
    (and dion/newton_schulz_triton.py:305-333 / `newton_schulz_triton` 336-374)
  * `zeropower_via_newtonschulz5_keller(G, steps=5, eps=1e-7)` -- reference dion/muon_reference.py:10-27
  * `ns_line_1(A)`, `ns_line_2(A, alpha, beta)`               -- reference dion/newton_schulz_triton.py:134-170, 261-302
"""
import torch
from torch import Tensor

from . import _lib

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

_workspace = _lib.Workspace()


def flat_coeffs(coeffs):
    return _lib.float_array([float(v) for abc in coeffs for v in abc])


def newton_schulz(
    G: Tensor,
    epsilon=1e-7,
    coeffs=NS_SCHEDULE_COEFFS,
    compute_dtype: torch.dtype = torch.bfloat16,
    faithful: bool = True,
) -> Tensor:
    """Orthogonalise the matrix (2-D) or batch of matrices (3-D) `G`; returns `compute_dtype`."""
    lib = _lib.load()
    _lib.require_gpu(G, "newton_schulz")
    if G.ndim not in (2, 3):
        raise ValueError(f"Expected a matrix or a batch of matrices, got {G.ndim}D")
    if G.dtype not in (torch.bfloat16, torch.float32):
        G = G.to(torch.float32)
    shape = G.shape
    G3 = G.reshape(-1, shape[-2], shape[-1]) if G.ndim == 2 else G
    if G3.stride(-1) != 1 or G3.stride(-2) != G3.size(-1) or (G3.size(0) > 1 and G3.stride(0) != G3.size(1) * G3.size(2)):
        G3 = G3.contiguous()
    if G3.size(1) % 8 or G3.size(2) % 8:
        # zero rows and columns stay zero through the iteration and change neither the norm nor the products
        padded = _lib.zero_padded(list(G3.unbind(0)), *_lib.padded_dims(G3.size(1), G3.size(2)))
        res = newton_schulz(padded, epsilon, coeffs, compute_dtype, faithful)
        return res[:, : G3.size(1), : G3.size(2)].reshape(shape)
    batch, m, n = G3.shape
    out = torch.empty((batch, m, n), dtype=compute_dtype, device=G.device)
    cd = _lib.dtype_code(compute_dtype)
    nbytes = lib.dion_amd_ns_workspace_bytes(batch, m, n, cd)
    ws = _workspace.get(nbytes, G.device)
    eps = float(epsilon)
    with torch.cuda.device(G.device):
        rc = lib.dion_amd_newton_schulz(
            G3.data_ptr(), _lib.dtype_code(G3.dtype), m * n, n,
            out.data_ptr(), m * n, n,
            batch, m, n, flat_coeffs(coeffs), len(coeffs), eps, cd, int(faithful),
            ws.data_ptr(), ws.numel(), _lib.stream_ptr(G.device),
        )
    _lib.check(rc, "dion_amd_newton_schulz")
    return out.reshape(shape)


def zeropower_via_newtonschulz5(G: Tensor, epsilon: float = 1e-7) -> Tensor:
    """Drop-in for reference dion/muon.py:620-647: schedule coefficients, bf16 result."""
    return newton_schulz(G, epsilon=epsilon, coeffs=NS_SCHEDULE_COEFFS)


def zeropower_via_newtonschulz5_keller(G: Tensor, steps: int = 5, eps: float = 1e-7) -> Tensor:
    """Drop-in for reference dion/muon_reference.py:10-27: fixed Keller coefficients, 2-D only."""
    assert len(G.shape) == 2, "Expected 2D tensor"
    return newton_schulz(G, epsilon=eps, coeffs=(NS_KELLER_COEFFS,) * steps)


def ns_line_1(A: Tensor, *, out: Tensor = None) -> Tensor:
    """A @ A.mT (reference dion/newton_schulz_triton.py:134-170)."""
    lib = _lib.load()
    _lib.require_gpu(A, "ns_line_1")
    A3 = (A if A.ndim == 3 else A.unsqueeze(0)).contiguous()
    batch, m, k = A3.shape
    if out is None:
        out = torch.empty((*A.shape[:-1], m), dtype=A.dtype, device=A.device)
    assert out.is_contiguous() and out.dtype == A.dtype
    with torch.cuda.device(A.device):
        rc = lib.dion_amd_syrk(A3.data_ptr(), m * k, k, out.data_ptr(), m * m, m, batch, m, k,
                               _lib.dtype_code(A.dtype), _lib.stream_ptr(A.device))
    _lib.check(rc, "dion_amd_syrk")
    return out


def ns_line_2(A: Tensor, alpha: float, beta: float, *, out: Tensor = None, faithful: bool = False) -> Tensor:
    """alpha * (A @ A.mT) + beta * A for symmetric A (reference dion/newton_schulz_triton.py:261-302)."""
    lib = _lib.load()
    _lib.require_gpu(A, "ns_line_2")
    A3 = (A if A.ndim == 3 else A.unsqueeze(0)).contiguous()
    batch, m, m2 = A3.shape
    assert m == m2, "Input must be square"
    if out is None:
        out = torch.empty_like(A, memory_format=torch.contiguous_format)
    assert out.is_contiguous() and out.dtype == A.dtype
    with torch.cuda.device(A.device):
        rc = lib.dion_amd_sym_poly(A3.data_ptr(), m * m, m, out.data_ptr(), m * m, m, batch, m,
                                   float(alpha), float(beta), _lib.dtype_code(A.dtype), int(faithful),
                                   _lib.stream_ptr(A.device))
    _lib.check(rc, "dion_amd_sym_poly")
    return out


def gemm(A: Tensor, B: Tensor, *, a_kstrided=False, b_kstrided=False, E: Tensor = None, s0=0.0, s1=1.0,
         out_dtype=None, out: Tensor = None, faithful=False) -> Tensor:
    """C = s0 * E + s1 * Aop @ Bop^T with Aop = A (M x K) or A^T when `a_kstrided` (A stored K x M);
    Bop = B (N x K) or B^T when `b_kstrided` (B stored K x N).  2-D or batched 3-D, contiguous."""
    lib = _lib.load()
    _lib.require_gpu(A, "gemm")
    A3 = (A if A.ndim == 3 else A.unsqueeze(0)).contiguous()
    B3 = (B if B.ndim == 3 else B.unsqueeze(0)).contiguous()
    batch = A3.size(0)
    K, M = (A3.size(1), A3.size(2)) if a_kstrided else (A3.size(2), A3.size(1))
    Kb, N = (B3.size(1), B3.size(2)) if b_kstrided else (B3.size(2), B3.size(1))
    assert K == Kb and B3.size(0) == batch
    out_dtype = out_dtype or A.dtype
    if out is None:
        out = torch.empty((batch, M, N), dtype=out_dtype, device=A.device)
    E3 = None
    if E is not None:
        E3 = (E if E.ndim == 3 else E.unsqueeze(0))
        assert E3.is_contiguous() and E3.dtype == out_dtype
    with torch.cuda.device(A.device):
        rc = lib.dion_amd_gemm(
            A3.data_ptr(), A3.size(1) * A3.size(2), A3.size(2), int(a_kstrided),
            B3.data_ptr(), B3.size(1) * B3.size(2), B3.size(2), int(b_kstrided),
            out.data_ptr(), M * N, N,
            E3.data_ptr() if E3 is not None else None, M * N, N,
            batch, M, N, K, _lib.dtype_code(A.dtype), _lib.dtype_code(out_dtype),
            _lib.EPI_AXPBY if E3 is not None else _lib.EPI_STORE, float(s0), float(s1), int(faithful),
            _lib.stream_ptr(A.device))
    _lib.check(rc, "dion_amd_gemm")
    return out if A.ndim == 3 else out[0]


def orthonormalize(P: Tensor, passes: int = 2, return_info: bool = False, qr_method: str = "rcqr",
                   sketch: Tensor = None):
    """Thin-QR Q factor of P (rows x r) or a batch of them on the device; counterpart of `orthogonalize`
    (reference dion/dion.py:1267-1308, dion/dion_reference.py:733-789), equal up to column signs.
    qr_method: "rcqr" -- CholeskyQR in fp32, in fp64 for the matrices whose measured defect asks for it, then a
    polishing pass; "qr" -- the fp64 pass for every matrix; "cqr" -- one fp32 CholeskyQR pass and nothing else
    (fp64 pass only if the factorisation fails).
    sketch: the reference's randomised Cholesky QR with this random sketch S (k x rows per matrix, P's dtype; see
    `dion_amd.dion.generate_random_sketch_matrix`), reference dion/dion.py:1287-1303; `qr_method` must be "rcqr"."""
    lib = _lib.load()
    _lib.require_gpu(P, "orthonormalize")
    P3 = (P if P.ndim == 3 else P.unsqueeze(0)).contiguous()
    batch, rows, r = P3.shape
    out = torch.empty_like(P3)
    info = torch.zeros(batch, dtype=torch.int32, device=P.device)
    if sketch is not None:
        if qr_method != "rcqr":
            raise ValueError("a sketch belongs to qr_method='rcqr'")
        S3 = (sketch if sketch.ndim == 3 else sketch.unsqueeze(0)).contiguous()
        if S3.dtype != P3.dtype or S3.shape[0] != batch or S3.shape[2] != rows:
            raise ValueError(f"sketch must be ({batch}, k, {rows}) in {P3.dtype}, got {tuple(S3.shape)} {S3.dtype}")
        k = S3.shape[1]
        ws = _workspace.get(lib.dion_amd_orthonormalize_sketch_workspace_bytes(batch, rows, r, k), P.device)
        with torch.cuda.device(P.device):
            rc = lib.dion_amd_orthonormalize_sketch(P3.data_ptr(), S3.data_ptr(), out.data_ptr(), _lib.dtype_code(P.dtype),
                                                    batch, rows, r, k, info.data_ptr(), ws.data_ptr(), ws.numel(),
                                                    _lib.stream_ptr(P.device))
        _lib.check(rc, "dion_amd_orthonormalize_sketch")
        out = out if P.ndim == 3 else out[0]
        return (out, info) if return_info else out
    nbytes = lib.dion_amd_orthonormalize_workspace_bytes(batch, rows, r)
    ws = _workspace.get(nbytes, P.device)
    with torch.cuda.device(P.device):
        rc = lib.dion_amd_orthonormalize_method(P3.data_ptr(), out.data_ptr(), _lib.dtype_code(P.dtype), batch, rows, r,
                                                passes, _lib.QR_METHODS[qr_method], info.data_ptr(), ws.data_ptr(),
                                                ws.numel(), _lib.stream_ptr(P.device))
    _lib.check(rc, "dion_amd_orthonormalize_method")
    out = out if P.ndim == 3 else out[0]
    return (out, info) if return_info else out
