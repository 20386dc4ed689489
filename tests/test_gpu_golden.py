"""The HIP path against the golden vectors produced by the reference implementation itself
(tests/golden/reference_vectors.npz), plus size-independent properties at the full benchmark shapes."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_fro

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLD)
    data = {k: z[k] for k in z.files}

    class Vectors(dict):
        def __getitem__(self, k):
            return torch.from_numpy(data[k].copy())

    return Vectors(data)


def _sign_align(a, ref):
    s = torch.sign((a.double() * ref.double()).sum(dim=0))
    s[s == 0] = 1
    return a.double() * s


@pytest.mark.parametrize("name", ["wide", "tall", "square", "batch"])
def test_ns_schedule_vs_reference_vectors(dev, gold, name):
    from dion_amd import zeropower_via_newtonschulz5

    got = zeropower_via_newtonschulz5(gold[f"ns_{name}_in"].to(dev))
    assert got.dtype == torch.bfloat16
    assert rel_fro(got, gold[f"ns_{name}_out"]) <= 2e-2


@pytest.mark.parametrize("name", ["wide", "tall"])
def test_ns_keller_vs_reference_vectors(dev, gold, name):
    from dion_amd.newton_schulz import zeropower_via_newtonschulz5_keller

    got = zeropower_via_newtonschulz5_keller(gold[f"keller_{name}_in"].to(dev), steps=5, eps=1e-7)
    assert rel_fro(got, gold[f"keller_{name}_out"]) <= 2e-2


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["tall", "wide", "square"])
def test_dion_two_steps_vs_reference_vectors(dev, gold, dt, name):
    from dion_amd import Dion, DionMixedPrecisionConfig

    mdt = torch.float32 if dt == "f32" else torch.bfloat16
    tag = f"dion_{dt}_{name}"
    p = torch.nn.Parameter(gold[tag + "_X0"].to(mdt).to(dev))
    q0 = gold[tag + "_Q0"]
    r = q0.shape[1]
    opt = Dion([p], rank_fraction=r / min(p.shape), lr=0.01, mu=0.95, weight_decay=0.01, epsilon=1e-8,
               mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=mdt, Q_dtype=torch.float32))
    st = opt._get_or_initialize_state(p, opt.param_groups[0])
    assert st["Q"].shape == q0.shape
    st["Q"].copy_(q0.to(dev))
    tol = 1e-4 if dt == "f32" else 1e-2
    for step in range(2):
        p.grad = gold[f"{tag}_G{step}"].to(mdt).to(dev)
        opt.step()
        assert rel_fro(st["momentum"], gold[f"{tag}_M{step + 1}"]) <= tol
        assert rel_fro(p.detach(), gold[f"{tag}_X{step + 1}"]) <= tol
        qref = gold[f"{tag}_Q{step + 1}"]
        qtol = tol * (50 if name == "square" else 3)  # full-rank square: conditioning-limited
        assert rel_fro(_sign_align(st["Q"].cpu(), qref), qref) <= qtol


def test_muon_step_vs_reference_vectors(dev, gold):
    """`Muon.step()` with the golden file's orthogonalised matrix plugged in through `newton_schulz_func`: momentum,
    the matrix handed to the hook, and the updated weights are the reference's own, bit for bit (the momentum pass
    and the weight update are element-wise with the reference's rounding points)."""
    from dion_amd import Muon

    for dt, dtype in (("bf16", torch.bfloat16), ("f32", torch.float32)):
        for nest in (True, False):
            tag = f"muon_{dt}_{'nesterov' if nest else 'plain'}"
            seen = []

            def hook(U, epsilon):
                seen.append(U.detach().float().cpu())
                return gold[f"muon_{dt}_Uo"].bfloat16().to(dev)

            p = torch.nn.Parameter(gold[f"muon_{dt}_X0"].to(dtype).to(dev))
            p.grad = gold[f"muon_{dt}_G"].to(dtype).to(dev)
            opt = Muon([p], lr=0.02, mu=0.95, weight_decay=0.01, nesterov=nest, newton_schulz_func=hook)
            opt.state[p]["momentum"] = gold[f"muon_{dt}_M0"].to(dtype).to(dev)
            opt.step()
            assert torch.equal(opt.state[p]["momentum"].float().cpu(), gold[tag + "_M1"])
            assert len(seen) == 1 and torch.equal(seen[0], gold[tag + "_U"])
            assert torch.equal(p.detach().float().cpu(), gold[f"muon_{dt}_X1"])
        # the fused path (library Newton-Schulz): same momentum
        p = torch.nn.Parameter(gold[f"muon_{dt}_X0"].to(dtype).to(dev))
        p.grad = gold[f"muon_{dt}_G"].to(dtype).to(dev)
        opt = Muon([p], lr=0.02, mu=0.95, weight_decay=0.01, nesterov=True)
        opt.state[p]["momentum"] = gold[f"muon_{dt}_M0"].to(dtype).to(dev)
        opt.step()
        assert torch.equal(opt.state[p]["momentum"].float().cpu(), gold[f"muon_{dt}_nesterov_M1"])


def test_ns_properties_at_llama8b_shape(dev):
    """4096 x 14336 (and its tall twin): transpose equivariance and near-orthonormal rows (Gram matrix of the
    first 1024 rows, a plain fp32 matmul on the CPU)."""
    from dion_amd import zeropower_via_newtonschulz5

    g = torch.Generator(device=dev).manual_seed(4)
    G = (torch.randn(4096, 14336, device=dev, generator=g) * 1e-3).bfloat16()
    X = zeropower_via_newtonschulz5(G)
    assert torch.equal(zeropower_via_newtonschulz5(G.mT.contiguous()), X.mT)
    Xs = X[:1024].float().cpu()
    gram = Xs @ Xs.T
    dev_from_i = (gram - torch.eye(1024)).norm().item() / 32.0   # / sqrt(rows)
    print(f"||X X^T - I||_F / sqrt(rows) = {dev_from_i:.3f}")
    assert dev_from_i < 0.1
    assert torch.isfinite(X.float()).all()


def test_dion_properties_at_llama70b_shape(dev):
    """One Dion step on a 28672 x 8192 bf16 matrix with r = 512: finite state, unit-norm Q columns, and the
    error-feedback identity ||B - M_new||_F = (1 - mu) ||P^T B||_F (P orthonormal) checked via
    ||B - M_new|| <= (1 - mu) ||B|| and the orthonormaliser's own Gram test at this size."""
    from dion_amd import Dion, DionMixedPrecisionConfig
    from dion_amd.newton_schulz import orthonormalize

    g = torch.Generator(device=dev).manual_seed(5)
    p = torch.nn.Parameter((torch.randn(28672, 8192, device=dev, generator=g) * 0.02).bfloat16())
    p.grad = (torch.randn(28672, 8192, device=dev, generator=g) * 1e-3).bfloat16()
    opt = Dion([p], rank_fraction=1.0 / 16, lr=0.01, mu=0.95, weight_decay=0.0,
               mixed_precision_config=DionMixedPrecisionConfig(momentum_dtype=torch.bfloat16, Q_dtype=torch.float32))
    x0 = p.detach().clone()
    opt.step()
    st = opt.state[p]
    assert st["Q"].shape == (8192, 512) and st["momentum"].dtype == torch.bfloat16
    assert torch.isfinite(st["momentum"].float()).all() and torch.isfinite(p.detach().float()).all()
    assert (st["Q"].double().norm(dim=0) - 1).abs().max().item() < 1e-2
    B = p.grad.float()                               # momentum started at zero: B = G
    removed = (B - st["momentum"].float()).norm().item()
    assert 0.0 < removed <= 0.05 * B.norm().item() * 1.05
    assert (p.detach().float() - x0.float()).abs().max().item() > 0
    assert int(torch.cat(list(opt.cholesky_info().values())).abs().sum().item()) == 0
    P = torch.randn(28672, 512, device=dev, generator=g)
    Qf = orthonormalize(P).cpu()
    assert ((Qf.T @ Qf) - torch.eye(512)).norm().item() <= 1e-3
