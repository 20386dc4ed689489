"""GPU parity of the GEMM entry points, called through the C ABI (ctypes).

Mirrors the reference's relational kernel tests (reference tests/test_newton_shultz.py:39-66:
shapes (256,256), (256,1024), batch 4, bf16 and fp32, allclose 5e-2) and adds tighter
Frobenius bounds, ragged tile edges and every operand layout.  The comparison products are
PyTorch matmuls on the CPU: the GPU side of these tests runs this library's kernels only.
"""
import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu

REF_TOL = 5e-2  # reference tests/test_newton_shultz.py:26-36


def _close(result, correct, tol=REF_TOL):
    result, correct = result.cpu(), correct.cpu()
    assert result.dtype == correct.dtype
    assert result.shape == correct.shape
    assert torch.allclose(result.float(), correct.float(), atol=tol, rtol=tol), (
        f"max-abs-diff {(result.float() - correct.float()).abs().max().item():.3e}"
    )


@pytest.mark.parametrize("m,n", [(256, 256), (256, 1024), (136, 200), (768, 3072)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ns_line_1(dev, m, n, dtype):
    from dion_amd.newton_schulz import ns_line_1

    torch.manual_seed(0)
    A = torch.randn(m, n, dtype=dtype, device=dev)
    Ac = A.cpu()
    ref = (Ac.double() @ Ac.double().mT)
    got = ns_line_1(A)
    _close(got, (Ac @ Ac.mT))
    assert rel_fro(got, ref) < (6e-3 if dtype == torch.bfloat16 else 1e-6)
    assert torch.equal(got, got.mT), "mirrored store must give an exactly symmetric result"

    Ab = torch.randn(4, m, n, dtype=dtype, device=dev)
    gotb = ns_line_1(Ab)
    Abc = Ab.cpu()
    _close(gotb, Abc @ Abc.mT)
    assert rel_fro(gotb, Abc.double() @ Abc.double().mT) < (6e-3 if dtype == torch.bfloat16 else 1e-6)


@pytest.mark.parametrize("m", [256, 392])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_ns_line_2(dev, m, dtype):
    from dion_amd.newton_schulz import ns_line_2

    torch.manual_seed(1)
    alpha, beta = torch.randn(1).item(), torch.randn(1).item()
    A = torch.randn(m, m, dtype=dtype, device=dev)
    A = (A + A.mT) / 2
    Ac = A.cpu()
    correct = alpha * (Ac @ Ac.mT) + beta * Ac
    _close(ns_line_2(A, alpha=alpha, beta=beta), correct, tol=REF_TOL * (4 if dtype == torch.bfloat16 else 1))
    ref64 = alpha * (Ac.double() @ Ac.double().mT) + beta * Ac.double()
    assert rel_fro(ns_line_2(A, alpha=alpha, beta=beta), ref64) < (6e-3 if dtype == torch.bfloat16 else 1e-6)

    Ab = torch.randn(4, m, m, dtype=dtype, device=dev)
    Ab = (Ab + Ab.mT) / 2
    Abc = Ab.cpu()
    ref64 = alpha * (Abc.double() @ Abc.double().mT) + beta * Abc.double()
    assert rel_fro(ns_line_2(Ab, alpha=alpha, beta=beta), ref64) < (6e-3 if dtype == torch.bfloat16 else 1e-6)


@pytest.mark.parametrize("a_ks", [False, True])
@pytest.mark.parametrize("b_ks", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K,batch", [(256, 384, 512, 1), (136, 72, 200, 3), (1024, 1024, 192, 2),
                                         # ragged dimension on a k-strided operand, everything else in whole tiles:
                                         # the direct-to-LDS K loop with a bounds-checked epilogue (Dion's rank 192)
                                         (768, 192, 768, 2), (192, 192, 1024, 2), (200, 320, 128, 1)])
def test_gemm_layouts(dev, a_ks, b_ks, dtype, M, N, K, batch):
    from dion_amd.newton_schulz import gemm

    torch.manual_seed(2)
    A = torch.randn(batch, K, M, dtype=dtype, device=dev) if a_ks else torch.randn(batch, M, K, dtype=dtype, device=dev)
    B = torch.randn(batch, K, N, dtype=dtype, device=dev) if b_ks else torch.randn(batch, N, K, dtype=dtype, device=dev)
    Aop = A.mT if a_ks else A
    Bop = B.mT if b_ks else B
    ref = Aop.cpu().double() @ Bop.cpu().double().mT
    got = gemm(A, B, a_kstrided=a_ks, b_kstrided=b_ks)
    assert got.shape == (batch, M, N) and got.dtype == dtype
    assert rel_fro(got, ref) < (5e-3 if dtype == torch.bfloat16 else 1e-6)
    # fused epilogue: C = s0 * E + s1 * A B^T, in place
    E = torch.randn(batch, M, N, dtype=dtype, device=dev)
    ref2 = 0.75 * E.cpu().double() - 1.5 * ref
    got2 = gemm(A, B, a_kstrided=a_ks, b_kstrided=b_ks, E=E, s0=0.75, s1=-1.5, out=E)
    assert got2.data_ptr() == E.data_ptr()
    assert rel_fro(got2, ref2) < (6e-3 if dtype == torch.bfloat16 else 1e-6)


def test_gemm_faithful_rounding_sequence(dev):
    """faithful=1 must reproduce torch's separate bf16 ops bit for bit when the matmul itself is exact
    (small integers: every product and partial sum is representable, so accumulation order is moot)."""
    from dion_amd.newton_schulz import gemm

    torch.manual_seed(3)
    M = N = 256
    K = 64
    A = torch.randint(-3, 4, (M, K), device=dev).to(torch.bfloat16)
    B = torch.randint(-3, 4, (N, K), device=dev).to(torch.bfloat16)
    E = torch.randn(M, N, device=dev).to(torch.bfloat16)
    c, b = 2.0315, -4.7750
    Ac, Bc = A.cpu(), B.cpu()
    want = b * E.cpu() + c * (Ac @ Bc.mT)  # each op rounds to bf16
    got = gemm(A, B, E=E, s0=b, s1=c, faithful=True)
    assert torch.equal(got.cpu(), want)
    # and the bf16-update-into-fp32-weights form (bf16 product scaled, added to fp32)
    E32 = torch.randn(M, N, device=dev)
    want32 = E32.cpu() * 0.9999 + (Ac @ Bc.mT) * -0.02
    got32 = gemm(A, B, E=E32.clone(), s0=0.9999, s1=-0.02, out_dtype=torch.float32, faithful=True)
    assert torch.equal(got32.cpu(), want32)


def test_alignment_is_rejected(dev):
    from dion_amd import _lib
    from dion_amd.newton_schulz import gemm

    A = torch.randn(64, 36, dtype=torch.bfloat16, device=dev)  # K = 36 is not a multiple of 8
    with pytest.raises(_lib.DionAmdError):
        gemm(A, A)
