"""The oracle against the golden vectors written by the reference implementation itself
(tests/golden/make_golden.py -> tests/golden/reference_vectors.npz).  CPU only."""
import os

import numpy as np
import pytest
import torch

from conftest import rel_fro

GOLD = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    z = np.load(GOLD)  # allow_pickle defaults to False
    data = {k: z[k] for k in z.files}

    class Vectors(dict):
        def __getitem__(self, k):  # fresh tensor every time: tests update their inputs in place
            return torch.from_numpy(data[k].copy())

    return Vectors(data)


def _sign_align(a, ref):
    s = torch.sign((a.double() * ref.double()).sum(dim=0))
    s[s == 0] = 1
    return a.double() * s


@pytest.mark.parametrize("name", ["wide", "tall", "square", "batch"])
def test_ns5_schedule_matches_reference(gold, name):
    from oracle import newton_schulz as O

    out = O.ns5(gold[f"ns_{name}_in"], epsilon=1e-7)
    ref = gold[f"ns_{name}_out"]
    assert out.dtype == torch.bfloat16 and out.shape == ref.shape
    # same ops on the same library: identical up to the BLAS thread partition
    assert rel_fro(out, ref) <= 1e-2
    assert (out.float() == ref).float().mean().item() > 0.5 or rel_fro(out, ref) < 5e-3


@pytest.mark.parametrize("name", ["wide", "tall"])
def test_ns5_keller_matches_reference(gold, name):
    from oracle import newton_schulz as O

    out = O.ns5_keller(gold[f"keller_{name}_in"], steps=5, eps=1e-7)
    assert rel_fro(out, gold[f"keller_{name}_out"]) <= 1.5e-2


@pytest.mark.parametrize("dt", ["bf16", "f32"])
@pytest.mark.parametrize("nesterov", [False, True])
def test_muon_passes_bit_exact(gold, dt, nesterov):
    from oracle import muon_step as O

    dtype = torch.bfloat16 if dt == "bf16" else torch.float32
    G, M = gold[f"muon_{dt}_G"].to(dtype), gold[f"muon_{dt}_M0"].to(dtype)
    U = O.muon_pre([G], [M], torch.tensor(0.95), nesterov)
    tag = f"muon_{dt}_{'nesterov' if nesterov else 'plain'}"
    assert torch.equal(M.float(), gold[tag + "_M1"]) and torch.equal(U[0].float(), gold[tag + "_U"])
    X = gold[f"muon_{dt}_X0"].to(dtype)
    lr, wd = torch.tensor(0.02), torch.tensor(0.01)
    O.muon_post([X], [gold[f"muon_{dt}_Uo"].bfloat16()], lr, O.adjust_lr(lr, X.shape, "spectral_norm"), wd)
    assert torch.equal(X.float(), gold[f"muon_{dt}_X1"])


@pytest.mark.parametrize("dt", ["f32", "bf16"])
@pytest.mark.parametrize("name", ["tall", "wide", "square"])
def test_dion_update_matches_reference(gold, dt, name):
    from oracle import dion_step as O

    mdt = torch.float32 if dt == "f32" else torch.bfloat16
    tag = f"dion_{dt}_{name}"
    X = gold[tag + "_X0"].to(mdt)
    M = torch.zeros_like(X)
    Q = gold[tag + "_Q0"].clone()
    gen = torch.Generator().manual_seed(123)  # a different sketch than the reference drew: M, X must not care
    tol = 2e-5 if dt == "f32" else 1e-2
    for step in range(2):
        G = gold[f"{tag}_G{step}"].to(mdt)
        O.dion_update(X, G, M, Q, lr=0.01, mu=0.95, weight_decay=0.01, epsilon=1e-8, generator=gen)
        assert rel_fro(M, gold[f"{tag}_M{step + 1}"]) <= tol
        assert rel_fro(X, gold[f"{tag}_X{step + 1}"]) <= tol
        qref = gold[f"{tag}_Q{step + 1}"]
        qtol = tol * (50 if name == "square" else 5)  # full-rank square: conditioning-limited
        assert rel_fro(_sign_align(Q, qref), qref) <= qtol
