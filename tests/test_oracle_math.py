"""What the mathematics fixes about the path, checked on the oracle (CPU only): closed forms,
invariants and brute-force roundings chosen so that a dropped term, a wrong sign or a
transposed operand fails one of them."""
import numpy as np
import pytest
import torch

from conftest import rel_fro


@pytest.mark.parametrize("shape", [(24, 40), (40, 24), (32, 32)])
@pytest.mark.parametrize("keller", [False, True])
def test_ns5_is_a_polynomial_of_the_singular_values(shape, keller):
    from oracle import newton_schulz as O

    torch.manual_seed(0)
    G = torch.randn(shape, dtype=torch.float64)
    coeffs = (O.NS_KELLER_COEFFS,) * 5 if keller else O.NS_SCHEDULE_COEFFS
    closed = O.ns5_closed_form(G, coeffs)
    assert rel_fro(O.ns5(G, coeffs=coeffs, compute_dtype=torch.float64), closed) < 1e-10
    assert rel_fro(O.ns5(G, coeffs=coeffs, compute_dtype=torch.float32), closed) < 1e-4
    assert rel_fro(O.ns5(G, coeffs=coeffs), closed) < 6e-2        # bf16 path: percent-level
    if keller:
        assert rel_fro(O.ns5_keller(G, compute_dtype=torch.float64), closed) < 1e-10
    # a wrong sign on b or a dropped c term changes the answer by O(1)
    bad = tuple((a, -b, c) for a, b, c in coeffs)
    assert rel_fro(O.ns5(G, coeffs=bad, compute_dtype=torch.float64), closed) > 0.5


def test_ns5_invariants():
    from oracle import newton_schulz as O

    torch.manual_seed(1)
    G = torch.randn(48, 96)
    X = O.ns5(G)
    assert X.dtype == torch.bfloat16
    assert torch.equal(O.ns5(G.T.contiguous()), X.T)             # NS(G^T) = NS(G)^T
    assert torch.equal(O.ns5(G * 8), X)                          # power-of-two scale invariance
    Gb = torch.stack([G, torch.randn(48, 96)])
    assert torch.equal(O.ns5(Gb)[0], X)                          # batch independence
    s = torch.linalg.svdvals(X.double())
    assert 0.9 < s.min() and s.max() < 1.1
    sk = torch.linalg.svdvals(O.ns5_keller(G).double())
    assert 0.6 < sk.min() and sk.max() < 1.2
    assert torch.count_nonzero(O.ns5(torch.zeros(8, 16))) == 0   # eps keeps 0 / 0 away


def test_bf16_rounding_helper_matches_torch():
    from oracle.bf16 import round_bf16

    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 100000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.005859375, 3.3895314e38], np.float32)])
    want = torch.from_numpy(x).bfloat16().float().numpy()
    assert np.array_equal(round_bf16(x), want)


@pytest.mark.parametrize("nesterov", [False, True])
def test_muon_passes_brute_force(nesterov):
    """Scalar restatement with explicit roundings: bf16 state rounds after every op, and the hyper-parameters
    are fp32 values (0.95f, not bf16(0.95))."""
    from oracle import muon_step as O
    from oracle.bf16 import round_bf16 as r

    rng = np.random.default_rng(2)
    g = r(rng.standard_normal(500).astype(np.float32) * 1e-3)
    m = r(rng.standard_normal(500).astype(np.float32) * 1e-3)
    mu = np.float32(0.95)
    m1 = r(r(m * mu) + g)
    u = r(r(m1 * mu) + g) if nesterov else m1
    M = torch.from_numpy(m).bfloat16().reshape(20, 25)
    U = O.muon_pre([torch.from_numpy(g).bfloat16().reshape(20, 25)], [M], torch.tensor(0.95), nesterov)
    assert np.array_equal(M.float().numpy().ravel(), m1)
    assert np.array_equal(U[0].float().numpy().ravel(), u)
    # post pass: X * (1 - lr wd) rounds, U * adjusted_lr rounds, the difference rounds
    x = r(rng.standard_normal(500).astype(np.float32) * 0.02)
    o = r(rng.standard_normal(500).astype(np.float32) * 0.1)
    lr, wd = np.float32(0.02), np.float32(0.01)
    alr = np.float32(lr * np.float32(np.sqrt(20 / 25)))
    want = r(r(x * np.float32(1 - lr * wd)) - r(o * alr))
    X = torch.from_numpy(x).bfloat16().reshape(20, 25)
    lr_t = torch.tensor(0.02)
    O.muon_post([X], [torch.from_numpy(o).bfloat16().reshape(20, 25)], lr_t, O.adjust_lr(lr_t, X.shape, "spectral_norm"),
                torch.tensor(0.01))
    assert np.array_equal(X.float().numpy().ravel(), want)


def test_adjust_lr_modes():
    from oracle import muon_step as O

    lr = torch.tensor(0.01)
    assert O.adjust_lr(lr, (4, 16), None) is lr
    assert abs(float(O.adjust_lr(lr, (4, 16), "spectral_norm")) - 0.01 * 0.5) < 1e-9
    assert abs(float(O.adjust_lr(lr, (4, 16), "rms_norm")) - 0.01 * 0.2 * 4.0) < 1e-9
    assert abs(float(O.adjust_lr(lr, (16, 4), "keller_muon")) - 0.01 * 2.0) < 1e-9
    assert abs(float(O.adjust_lr(lr, (4, 16), "keller_muon")) - 0.01) < 1e-9
    with pytest.raises(ValueError):
        O.adjust_lr(lr, (4, 16), "nope")


@pytest.mark.parametrize("shape,r", [((96, 64), 16), ((64, 96), 16)])
def test_dion_update_identities(shape, r):
    from oracle import dion_step as O

    torch.manual_seed(3)
    X0 = torch.randn(shape, dtype=torch.float64) * 0.02
    G = torch.randn(shape, dtype=torch.float64) * 1e-3
    M0 = torch.randn(shape, dtype=torch.float64) * 1e-3
    Q0 = torch.randn(min(shape), r, dtype=torch.float64)
    lr, mu, wd = 0.01, 0.95, 0.1
    X, M, Q = X0.clone(), M0.clone(), Q0.clone()
    P, R = O.dion_update(X, G, M, Q, lr, mu, wd)
    B = M0 + G
    Bv = B.T if shape[0] < shape[1] else B
    eye = torch.eye(r, dtype=torch.float64)
    assert (P.T @ P - eye).norm() < 1e-5                                    # orthonormal
    Pq, _ = torch.linalg.qr(Bv @ Q0)
    assert ((P @ P.T) - (Pq @ Pq.T)).norm() < 1e-5                          # spans col(B Q)
    assert rel_fro(R, Bv.T @ P) < 1e-6                                      # R = B^T P
    low = P @ R.T
    low = low.T if shape[0] < shape[1] else low
    assert rel_fro(M, B - (1 - mu) * low) < 1e-6                            # error feedback
    assert ((Q.norm(dim=0) - 1).abs().max()) < 1e-6                         # unit columns
    upd = P @ Q.T
    upd = upd.T if shape[0] < shape[1] else upd
    want = (1 - lr * wd) * X0 - (shape[0] / shape[1]) ** 0.5 * lr * upd
    assert rel_fro(X, want) < 1e-6                                          # weight update
    # M and X do not depend on the sketch seed nor on column signs of P (Q flips sign with P)
    flip = torch.ones(r, dtype=torch.float64)
    flip[::2] = -1
    X2, M2, Q2 = X0.clone(), M0.clone(), Q0.clone()
    O.dion_update(X2, G, M2, Q2, lr, mu, wd, orth=lambda p: O.orthogonalize(p, generator=torch.Generator().manual_seed(9)) * flip)
    sgn = torch.sign((Q2 * Q).sum(dim=0))
    assert rel_fro(M2, M) < 1e-6 and rel_fro(X2, X) < 1e-6 and rel_fro(Q2 * sgn, Q) < 1e-5


def test_dion_full_rank_and_zero_cases():
    from oracle import dion_step as O

    torch.manual_seed(4)
    n = 48
    X, G, M = torch.randn(n, n, dtype=torch.float64), torch.randn(n, n, dtype=torch.float64), torch.zeros(n, n, dtype=torch.float64)
    Q = torch.randn(n, n, dtype=torch.float64)
    O.dion_update(X, G, M, Q, 0.01, 0.95, 0.0)
    assert rel_fro(M, 0.95 * G) < 1e-6          # full rank: P P^T = I, so M_new = mu * B
    # all-zero gradient and momentum: P = 0, R = Q_init, M stays 0, X only decays
    X = torch.randn(32, 16, dtype=torch.float64)
    X0, Q = X.clone(), torch.randn(16, 4, dtype=torch.float64)
    Q0 = Q.clone()
    M = torch.zeros(32, 16, dtype=torch.float64)
    P, R = O.dion_update(X, torch.zeros(32, 16, dtype=torch.float64), M, Q, 0.01, 0.95, 0.1)
    assert torch.count_nonzero(P) == 0 and torch.count_nonzero(M) == 0
    assert rel_fro(X, X0 * (1 - 0.01 * 0.1)) < 1e-6
    assert rel_fro(Q, Q0 / Q0.norm(dim=0, keepdim=True)) < 1e-6
    assert O.rank_of(768, 3072, 0.25) == 192 and O.rank_of(100, 60, 0.3, 8) == 24 and O.rank_of(10, 10, 1.0, 16) == 10


@pytest.mark.parametrize("shape", [(96, 64), (64, 96)])
@pytest.mark.parametrize("qr_method", ["qr", "cqr", "rcqr"])
def test_dion_reference_update_power_iterations(shape, qr_method):
    """`dion_update_reference`: one iteration equals `dion_update`; k iterations give the projector onto
    col(B (B^T B)^(k-1) Q) in the error feedback and the update -- the closed form, evaluated here with
    a Householder QR in fp64 (a dropped or repeated iteration, or a missing transpose, changes the subspace)."""
    from oracle import dion_step as O

    torch.manual_seed(8)
    r = 12
    X0 = torch.randn(shape, dtype=torch.float64) * 0.02
    G = torch.randn(shape, dtype=torch.float64) * 1e-3
    M0 = torch.randn(shape, dtype=torch.float64) * 1e-3
    Q0 = torch.randn(min(shape), r, dtype=torch.float64)
    lr, mu, wd, eps = 0.01, 0.95, 0.1, 1e-8
    Xa, Ma, Qa = X0.clone(), M0.clone(), Q0.clone()
    O.dion_update(Xa, G, Ma, Qa, lr, mu, wd, eps)
    Xb, Mb = X0.clone(), M0.clone()
    Qb = O.dion_update_reference(Xb, G, Mb, Q0.clone(), lr, mu, wd, eps, power_iters=1, qr_method=qr_method,
                                 generator=torch.Generator().manual_seed(1))
    sgn = torch.sign((Qa * Qb).sum(dim=0))
    assert rel_fro(Mb, Ma) < 1e-6 and rel_fro(Xb, Xa) < 1e-6 and rel_fro(Qb * sgn, Qa) < 1e-5
    B = M0 + G
    Bv = B.T if shape[0] < shape[1] else B
    for k in (2, 3):
        X, M = X0.clone(), M0.clone()
        Qn = O.dion_update_reference(X, G, M, Q0.clone(), lr, mu, wd, eps, power_iters=k, qr_method=qr_method,
                                     generator=torch.Generator().manual_seed(1))
        K = Bv @ Q0
        for _ in range(k - 1):
            K = Bv @ (Bv.T @ torch.linalg.qr(K)[0])   # re-orthonormalised: the powers of B^T B are ill-conditioned
        Pk = torch.linalg.qr(K)[0]
        low = Pk @ (Pk.T @ Bv)
        low = low.T if shape[0] < shape[1] else low
        assert rel_fro(M, B - (1 - mu) * low) < 1e-6, (k, qr_method)
        Rk = Bv.T @ Pk
        Qk = Rk / (Rk.norm(dim=0, keepdim=True) + eps)
        upd = Pk @ Qk.T
        upd = upd.T if shape[0] < shape[1] else upd
        assert rel_fro(X, (1 - lr * wd) * X0 - (shape[0] / shape[1]) ** 0.5 * lr * upd) < 1e-6, (k, qr_method)
        s2 = torch.sign((Qn * Qk).sum(dim=0))
        assert rel_fro(Qn * s2, Qk) < 1e-5


def test_orthogonalize_variants_agree():
    from oracle import dion_step as O

    torch.manual_seed(5)
    P = torch.randn(200, 24)
    ref = O.orthogonalize_variant(P, "qr")
    for method in ("cqr", "rcqr"):
        Qm = O.orthogonalize_variant(P, method, generator=torch.Generator().manual_seed(0))
        s = torch.sign((Qm * ref).sum(0))
        assert rel_fro(Qm * s, ref) < 1e-4
    wide = torch.randn(1, 16, 24)
    Qw = O.orthogonalize(wide)                 # rows <= cols: Householder branch
    assert (Qw[0].T @ Qw[0]).shape == (16, 16) or Qw.shape == (1, 16, 16)


def test_scalar_opts_match_closed_forms():
    """Lion / AdamW oracle (reference dion/scalar_opts.py:89-187) against the textbook forms in fp64."""
    from oracle.scalar_opts import adamw_update_foreach, lion_update_foreach

    torch.manual_seed(0)
    x, g = torch.randn(50, dtype=torch.float64), torch.randn(50, dtype=torch.float64)
    m, v = torch.randn(50, dtype=torch.float64) * 0.1, torch.rand(50, dtype=torch.float64) * 0.1
    lr, b1, b2, wd, eps, step = 0.01, 0.9, 0.95, 0.1, 1e-8, 3
    m1 = b1 * m + (1 - b1) * g
    v1 = b2 * v + (1 - b2) * g * g
    want = x * (1 - lr * wd) - lr * (m1 / (1 - b1**step)) / ((v1 / (1 - b2**step)).sqrt() + eps)
    X, M, V = [x.clone()], [m.clone()], [v.clone()]
    t = lambda z: torch.tensor(z, dtype=torch.float64)  # noqa: E731
    adamw_update_foreach(X, [g], M, V, t(lr), t(b1), t(b2), t(wd), t(step), t(eps))
    assert torch.allclose(X[0], want, rtol=1e-9) and torch.allclose(M[0], m1) and torch.allclose(V[0], v1)
    want = x * (1 - lr * wd) - lr * torch.sign(b1 * m + (1 - b1) * g)
    X, M = [x.clone()], [m.clone()]
    lion_update_foreach(X, [g], M, t(lr), t(b1), t(b2), t(wd))
    assert torch.allclose(X[0], want, rtol=1e-12) and torch.allclose(M[0], b2 * m + (1 - b2) * g)


def test_scalar_opts_bf16_rounding_points():
    """In bf16 every tensor op of the reference rounds once; the oracle must equal an fp32 evaluation of the same
    sequence with an explicit bf16 rounding after each op (the 0-dim lerp weights 0.1 / 0.05 are cast to bf16 first
    and use the `start + w*(end-start)` branch with a fused multiply-add, as ATen's kernel does)."""
    from oracle.scalar_opts import adamw_update_foreach, lion_update_foreach

    r = lambda z: z.to(torch.bfloat16).to(torch.float32)  # noqa: E731
    torch.manual_seed(1)
    n = 4096
    x0, g0 = r(torch.randn(n)), r(torch.randn(n) * 0.1)
    m0, v0 = r(torch.randn(n) * 0.1), r(torch.rand(n) * 0.01)
    f = lambda z: torch.tensor(z, dtype=torch.float32)  # noqa: E731
    lr, b1, b2, wd, eps, step = f(0.01), f(0.9), f(0.95), f(0.1), 1e-8, 2
    w1, w2, decay = 1 - b1, 1 - b2, 1 - lr * wd

    def lerp(s, e, w):
        return r(torch.addcmul(s.double(), (e - s).double(), r(w).double()).float())  # one rounding of the fma in fp32

    # Lion
    u = torch.sign(lerp(m0, g0, w1))
    m1 = lerp(m0, g0, w2)
    x1 = r(r(x0 * decay) - r(u * lr))
    X, M = [x0.bfloat16()], [m0.bfloat16()]
    lion_update_foreach(X, [g0.bfloat16()], M, lr, b1, b2, wd)
    assert torch.equal(M[0].float(), m1)
    assert (X[0].float() != x1).float().mean() < 1e-3  # double-rounding ties of the fp64 stand-in for the fma
    # AdamW
    m1 = lerp(m0, g0, w1)
    v1 = lerp(v0, r(g0 * g0), w2)
    den = r(r(r(v1.sqrt()) / (1 - b2**step).sqrt()) + eps)
    x1 = r(r(x0 * decay) - r(r(m1 / den) * (lr / (1 - b1**step))))
    X, M, V = [x0.bfloat16()], [m0.bfloat16()], [v0.bfloat16()]
    adamw_update_foreach(X, [g0.bfloat16()], M, V, lr, b1, b2, wd, step, eps)
    assert torch.equal(M[0].float(), m1) and torch.equal(V[0].float(), v1)
    assert (X[0].float() != x1).float().mean() < 1e-3


def test_sketched_orthogonalize_is_the_thin_qr_factor_whatever_the_sketch():
    """`orthogonalize` with an injected sketch (reference dion/dion.py:1287-1303): in exact arithmetic the result is
    the thin-QR Q factor of P for ANY full-rank sketch -- S only preconditions.  Pinned against Householder QR in
    fp64 (a library routine) up to column signs, for two different sketches and for a deliberately poor one
    (a dropped `R1^-1`, a transposed solve or a missing second factorisation all fail this)."""
    from oracle import dion_step as O

    torch.manual_seed(12)
    rows, r = 384, 48
    U, _ = torch.linalg.qr(torch.randn(rows, r, dtype=torch.float64))
    V, _ = torch.linalg.qr(torch.randn(r, r, dtype=torch.float64))
    P = ((U * torch.logspace(0, -3, r, dtype=torch.float64)) @ V.T).float().unsqueeze(0)      # cond 1e3
    Qh, _ = torch.linalg.qr(P[0].double())
    g = torch.Generator().manual_seed(1)
    for trial in range(3):
        S = O.sketch_matrix(P, 1.25, g)
        assert S.shape == (1, 128, rows)
        if trial == 2:
            S = S * torch.logspace(0, -2, 128).view(1, -1, 1)      # a badly scaled sketch still spans enough
        Q = O.orthogonalize(P, sketch=S)[0].double()
        sgn = torch.sign((Q * Qh).sum(dim=0))
        assert ((Q * sgn - Qh).norm() / Qh.norm()).item() <= 2e-4
        assert (Q.T @ Q - torch.eye(r, dtype=torch.float64)).norm().item() <= 1e-4
    # drawing from a generator and injecting the same draw are the same thing
    a = O.orthogonalize(P, generator=torch.Generator().manual_seed(7))
    b = O.orthogonalize(P, sketch=O.sketch_matrix(P, 1.25, torch.Generator().manual_seed(7)))
    assert torch.equal(a, b)
