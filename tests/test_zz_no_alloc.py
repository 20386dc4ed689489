"""The allocation-free Newton-Schulz entry point (`dion_amd_newton_schulz_static`: working matrices in a
device array that is part of the library image) against `dion_amd_newton_schulz` with a caller-owned workspace,
through the C ABI.  Both run the same kernels in the same order, so the results must be identical bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(lib, _lib, G, compute_dtype, dev):
    from dion_amd.newton_schulz import NS_SCHEDULE_COEFFS, flat_coeffs

    batch, m, n = G.shape
    cd = _lib.dtype_code(compute_dtype)
    coeffs = flat_coeffs(NS_SCHEDULE_COEFFS)
    ref = torch.empty((batch, m, n), dtype=compute_dtype, device=dev)
    ws = torch.empty(lib.dion_amd_ns_workspace_bytes(batch, m, n, cd), dtype=torch.uint8, device=dev)
    rc = lib.dion_amd_newton_schulz(G.data_ptr(), _lib.dtype_code(G.dtype), m * n, n, ref.data_ptr(), m * n, n,
                                    batch, m, n, coeffs, 5, 1e-7, cd, 1, ws.data_ptr(), ws.numel(), _lib.stream_ptr(dev))
    assert rc == 0, rc
    got = torch.full((batch, m, n), float("nan"), dtype=compute_dtype, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    rc = lib.dion_amd_newton_schulz_static(G.data_ptr(), _lib.dtype_code(G.dtype), m * n, n, got.data_ptr(), m * n, n,
                                           batch, m, n, coeffs, 5, 1e-7, cd, 1, _lib.stream_ptr(dev))
    assert rc == 0, rc
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    return got, ref


def test_static_newton_schulz_equals_workspace_version_twice(dev):
    from dion_amd import _lib

    lib = _lib.load()
    assert lib.dion_amd_static_scratch_bytes() == 32 << 20
    gen = torch.Generator().manual_seed(9)
    # first call: a batch that needs three chunks of the array (768 x 3072: 11.8 MB per matrix), tall orientation
    G1 = (torch.randn((5, 3072, 768), generator=gen) * 1e-3).bfloat16().to(dev)
    got, ref = _both(lib, _lib, G1, torch.bfloat16, dev)
    assert torch.isfinite(got.float()).all() and torch.equal(got, ref)
    # second call, smaller input (the array still holds the first call's matrices), fp32 gradients and fp32 iteration
    G2 = (torch.randn((3, 136, 200), generator=gen)).to(dev)
    got, ref = _both(lib, _lib, G2, torch.float32, dev)
    assert torch.isfinite(got).all() and torch.equal(got, ref)
    # and a bf16 one after it, smaller again
    G3 = (torch.randn((1, 64, 128), generator=gen)).bfloat16().to(dev)
    got, ref = _both(lib, _lib, G3, torch.bfloat16, dev)
    assert torch.equal(got, ref)


def test_static_newton_schulz_rejects_what_does_not_fit(dev):
    from dion_amd import _lib
    from dion_amd.newton_schulz import NS_SCHEDULE_COEFFS, flat_coeffs

    lib = _lib.load()
    m, n = 4096, 4096   # 2 x 33.6 MB + 2 x 33.6 MB per matrix: beyond the 32 MiB array
    assert lib.dion_amd_ns_workspace_bytes(1, m, n, _lib.BF16) > lib.dion_amd_static_scratch_bytes()
    G = torch.zeros((1, m, n), dtype=torch.bfloat16, device=dev)
    out = torch.full_like(G, 7.0)
    rc = lib.dion_amd_newton_schulz_static(G.data_ptr(), _lib.BF16, m * n, n, out.data_ptr(), m * n, n, 1, m, n,
                                           flat_coeffs(NS_SCHEDULE_COEFFS), 5, 1e-7, _lib.BF16, 1, _lib.stream_ptr(dev))
    assert rc == -5
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())   # nothing was launched
    with pytest.raises(_lib.DionAmdError, match="limit"):
        _lib.check(rc, "dion_amd_newton_schulz_static")
