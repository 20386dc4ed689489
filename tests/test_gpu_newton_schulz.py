"""GPU parity of the Newton-Schulz path against the CPU oracle, through the C ABI."""
import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2   # bf16 NS vs the reference bf16 path, relative Frobenius (north star)
FP32_TOL = 1e-4   # fp32 NS vs an fp32/fp64 evaluation of the same recurrence


def _orth_err(X):
    X = X.double().cpu()
    if X.size(-2) > X.size(-1):
        X = X.mT
    s = torch.linalg.svdvals(X)
    return s.min().item(), s.max().item()


@pytest.mark.parametrize("m,n", [(768, 3072), (3072, 768), (768, 768), (256, 1024), (256, 256), (1024, 4096), (136, 200),
                                 (100, 301), (301, 100), (77, 77), (64, 27)])
def test_ns_bf16_schedule_vs_oracle(dev, m, n):
    from dion_amd import zeropower_via_newtonschulz5
    from oracle import newton_schulz as O

    torch.manual_seed(0)
    G = torch.randn(m, n)
    ref = O.ns5(G)  # bf16 op-by-op reference path on CPU
    got = zeropower_via_newtonschulz5(G.to(dev))
    assert got.dtype == torch.bfloat16 and got.shape == (m, n)
    err = rel_fro(got, ref)
    print(f"ns bf16 schedule {m}x{n}: rel fro {err:.3e}")
    assert err <= BF16_TOL
    lo, hi = _orth_err(got)
    rlo, rhi = _orth_err(ref)  # singular-value range of the reference result (square inputs keep values near 0)
    assert abs(lo - rlo) < 0.05 and abs(hi - rhi) < 0.05
    if max(m, n) >= 2 * min(m, n):
        assert 0.9 < lo and hi < 1.1  # schedule coefficients land in ~[0.97, 1.035]


def test_ns_config1_keller(dev):
    """CPU-runnable configuration: one 768x3072 fp32 N(0,1) seed-0 matrix, Keller coefficients, eps 1e-7."""
    from dion_amd.newton_schulz import zeropower_via_newtonschulz5_keller
    from oracle import newton_schulz as O

    torch.manual_seed(0)
    G = torch.randn(768, 3072)
    for src in (G, G.T.contiguous()):
        ref = O.ns5_keller(src, steps=5, eps=1e-7)
        got = zeropower_via_newtonschulz5_keller(src.to(dev), steps=5, eps=1e-7)
        err = rel_fro(got, ref)
        print(f"ns keller {tuple(src.shape)}: rel fro {err:.3e}")
        assert err <= BF16_TOL
        lo, hi = _orth_err(got)
        assert 0.6 < lo and hi < 1.2  # Keller coefficients: ~[0.68, 1.14]


@pytest.mark.parametrize("m,n", [(256, 1024), (768, 768), (1024, 256)])
def test_ns_fp32_mode(dev, m, n):
    from dion_amd.newton_schulz import newton_schulz, NS_SCHEDULE_COEFFS, NS_KELLER_COEFFS
    from oracle import newton_schulz as O

    torch.manual_seed(1)
    G = torch.randn(m, n)
    for coeffs in (NS_SCHEDULE_COEFFS, (NS_KELLER_COEFFS,) * 5):
        ref = O.ns5(G, coeffs=coeffs, compute_dtype=torch.float64)
        got = newton_schulz(G.to(dev), coeffs=coeffs, compute_dtype=torch.float32)
        assert got.dtype == torch.float32
        err = rel_fro(got, ref)
        print(f"ns fp32 {m}x{n}: rel fro {err:.3e}")
        assert err <= FP32_TOL


def test_ns_batched_and_input_dtypes(dev):
    from dion_amd import zeropower_via_newtonschulz5
    from oracle import newton_schulz as O

    torch.manual_seed(2)
    G = torch.randn(4, 256, 1024) * 1e-3
    ref = O.ns5(G)
    got = zeropower_via_newtonschulz5(G.to(dev))
    assert got.shape == G.shape
    for b in range(4):
        assert rel_fro(got[b], ref[b]) <= BF16_TOL
    # batch independence: each matrix alone gives the same bits as in the batch
    alone = zeropower_via_newtonschulz5(G[2].to(dev))
    assert torch.equal(alone, got[2])
    # bf16 input and a non-contiguous (.mT) view
    gb = G[0].to(dev).bfloat16()
    assert rel_fro(zeropower_via_newtonschulz5(gb), O.ns5(G[0].bfloat16())) <= BF16_TOL
    assert rel_fro(zeropower_via_newtonschulz5(gb.mT), O.ns5(G[0].bfloat16().mT)) <= BF16_TOL


def test_ns_invariants_large(dev):
    """Size-independent properties at a benchmark shape too large for the CPU oracle in a test:
    NS(G^T) = NS(G)^T, NS(2^k G) = NS(G) exactly, singular values pulled into ~[0.9, 1.1]."""
    from dion_amd import zeropower_via_newtonschulz5

    torch.manual_seed(4)
    G = (torch.randn(2048, 7168, device=dev) * 1e-3).bfloat16()
    X = zeropower_via_newtonschulz5(G)
    assert torch.equal(zeropower_via_newtonschulz5(G.mT.contiguous()), X.mT)
    assert torch.equal(zeropower_via_newtonschulz5(G * 4), X)
    s = torch.linalg.svdvals(X.float())
    assert 0.9 < s.min().item() and s.max().item() < 1.1


def test_ns_zero_matrix(dev):
    from dion_amd import zeropower_via_newtonschulz5

    Z = torch.zeros(256, 512, device=dev)
    out = zeropower_via_newtonschulz5(Z)
    assert torch.count_nonzero(out) == 0 and torch.isfinite(out.float()).all()


@pytest.mark.gpu
@pytest.mark.parametrize("m,n", [(256, 256), (256, 1024)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_newton_schulz_triton_matches_eager_rounding(dev, m, n, dtype):
    """The reference's own relational test (tests/test_newton_shultz.py:77-88): the fused-epilogue variant against
    the op-by-op variant, atol = rtol = 5e-2, 2-D and batch of 4, through the reference's import path."""
    from dion_amd.newton_schulz_triton import newton_schulz_triton, zeropower_via_newtonschulz5
    g = torch.Generator().manual_seed(11)
    for shape in ((m, n), (4, m, n)):
        G = torch.randn(*shape, generator=g).to(dtype).to(dev)
        a, b = newton_schulz_triton(G), zeropower_via_newtonschulz5(G)
        assert a.dtype == b.dtype == torch.bfloat16 and a.shape == b.shape == G.shape
        assert torch.allclose(a.float(), b.float(), atol=5e-2, rtol=5e-2), (a.float() - b.float()).abs().max()


@pytest.mark.gpu
def test_muon_reference_import_path(dev):
    from dion_amd.muon_reference import zeropower_via_newtonschulz5 as keller
    from dion_amd.newton_schulz import NS_KELLER_COEFFS, newton_schulz
    G = torch.randn(128, 256, generator=torch.Generator().manual_seed(12)).to(dev)
    assert torch.equal(keller(G, steps=3), newton_schulz(G, epsilon=1e-7, coeffs=(NS_KELLER_COEFFS,) * 3))
    with pytest.raises(AssertionError):
        keller(G.unsqueeze(0))


@pytest.mark.parametrize("shape", [(768, 768), (256, 1024), (1024, 256), (3, 384, 640)])
def test_frobenius_normalisation_is_bit_exact(dev, shape):
    """Zero iterations leave X / (||X||_F + eps) (reference dion/muon.py:633-638): same bf16 values as the op-by-op
    evaluation, division included, whenever the two norms round to the same bf16 number (sums in another order)."""
    from dion_amd.newton_schulz import newton_schulz
    from oracle import newton_schulz as ON

    torch.manual_seed(9)
    G = torch.randn(shape)
    got = newton_schulz(G.to(dev), coeffs=()).cpu()
    ref = ON.ns5(G, coeffs=())
    assert got.dtype == torch.bfloat16 and got.shape == ref.shape
    mism = (got != ref).float().mean().item()
    print(f"normalisation {shape}: {mism:.2e} of the elements differ")
    X = G.bfloat16()
    n_ref = X.norm(dim=(-2, -1)) + 1e-7
    n_f64 = (X.double().norm(dim=(-2, -1)).float().bfloat16() + 1e-7)
    if torch.equal(n_ref, n_f64):
        assert mism == 0.0
    else:
        assert rel_fro(got, ref) <= 8e-3   # the norms themselves differ by one bf16 ulp
